// Device helpers shared by the sparse and dense attention kernels: wavefront reductions, the
// work-group -> XCD mapping and the register-level 32x32 MFMA tile operations.
#pragma once
#include <hip/hip_runtime.h>

namespace spion {

// =================================================================================================
// wavefront helpers
// =================================================================================================
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Row of the 32x32 MFMA accumulator held in register r of a lane in half h (lane / 32); the column
// is lane % 32.
__device__ __forceinline__ int acc_row(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

// Work-group id -> work item, so that consecutive work items (same head) run on the same XCD and
// share its L2: the hardware deals work-groups round-robin over the 8 XCDs.
__device__ __forceinline__ int xcd_remap(int pid, int total) {
    constexpr int XCDS = 8;
    if (total % XCDS) return pid;
    return (pid % XCDS) * (total / XCDS) + pid / XCDS;
}

// =================================================================================================
// MFMA tile operations
// =================================================================================================
// Operand conventions for v_mfma_f32_32x32x2_f32 (D = A.B + C, A 32x2, B 2x32):
//   lane l supplies A[l%32][l/32] and B[l/32][l%32]; register r of the 16-register accumulator of
//   lane l holds D[acc_row(r, l/32)][l%32].
// A contraction over the head dimension is a chain of D/2 such instructions; which feature index t a
// (step s, half h) slot stands for is free as long as A and B agree -- here t = h*(D/2) + s, so that a
// lane reads D/2 consecutive floats of a row-major row.
// A contraction over the 32 keys/queries of a tile is a chain of 16 instructions in which slot (s, h)
// stands for tile row acc_row(s, h): the accumulator of the first product is then already the A
// operand of the second one, register for register, and nothing goes through LDS.

template <int D>
__device__ __forceinline__ void load_rows(const float* __restrict__ X, int row0, int li, int h, float (&x)[D / 2]) {
    const float4* p = reinterpret_cast<const float4*>(X + (size_t)(row0 + li) * D + h * (D / 2));
#pragma unroll
    for (int q = 0; q < D / 8; ++q) {
        float4 v = p[q];
        x[4 * q + 0] = v.x;
        x[4 * q + 1] = v.y;
        x[4 * q + 2] = v.z;
        x[4 * q + 3] = v.w;
    }
}

template <int D>
__device__ __forceinline__ void load_cols(const float* __restrict__ Xt, int L, int col0, int li, int h,
                                          float (&x)[D / 2]) {
    const float* p = Xt + (size_t)(h * (D / 2)) * L + col0 + li;
#pragma unroll
    for (int s = 0; s < D / 2; ++s) x[s] = p[(size_t)s * L];
}

template <int D>
__device__ __forceinline__ f32x16 mma_feat(const float (&a)[D / 2], const float (&b)[D / 2]) {
    f32x16 acc = {0};
#pragma unroll
    for (int s = 0; s < D / 2; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
    return acc;
}

// out[c] += W(32x32, as accumulator-layout registers w[16]) . X[row0 .. row0+32)[c*32 .. c*32+32)
template <int D>
__device__ __forceinline__ void mma_tile(const float (&w)[16], const float* __restrict__ X, int row0, int li,
                                         int h, f32x16 (&out)[D / 32]) {
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        float x[16];
#pragma unroll
        for (int s = 0; s < 16; ++s) x[s] = X[(size_t)(row0 + acc_row(s, h)) * D + c * 32 + li];
#pragma unroll
        for (int s = 0; s < 16; ++s) out[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(w[s], x[s], out[c], 0, 0, 0);
    }
}

// out[c] (+)= X^T-tile . W for operands stored feature-major (Xt [D][ld], the dense-phase layout):
// result row = feature c*32 + (lane%32 as A row), column = the accumulator column of W.  W enters as
// the B operand (slot (s, h) = tile row acc_row(s, h)), Xt as the A operand read with float4 loads.
template <int D>
__device__ __forceinline__ void mma_tile_t(const float (&w)[16], const float* __restrict__ Xt, size_t ld, int col0,
                                           int li, int h, f32x16 (&out)[D / 32]) {
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        float x[16];
        const float* p = Xt + (size_t)(c * 32 + li) * ld + col0 + 4 * h;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float4 v = *reinterpret_cast<const float4*>(p + 8 * g);
            x[4 * g + 0] = v.x;
            x[4 * g + 1] = v.y;
            x[4 * g + 2] = v.z;
            x[4 * g + 3] = v.w;
        }
#pragma unroll
        for (int s = 0; s < 16; ++s) out[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(x[s], w[s], out[c], 0, 0, 0);
    }
}

// Sum the per-wave accumulators of a work-group and store the result tile(s).
//   TRANS == false: accumulator c holds rows row0+acc_row of a row-major [.][D] array, columns c*32+lane%32.
//   TRANS == true : accumulator c holds rows c*32+acc_row of a feature-major [D][ld] array, columns row0+lane%32.
template <int D, int WAVES, bool TRANS = false>
__device__ __forceinline__ void reduce_store(f32x16 (&acc)[D / 32], float* __restrict__ out, int row0, int w,
                                             int li, int h, float* __restrict__ lds, size_t ld = D) {
    constexpr int NC = D / 32;
    auto addr = [&](int c, int r) -> size_t {
        return TRANS ? (size_t)(c * 32 + acc_row(r, h)) * ld + row0 + li
                     : (size_t)(row0 + acc_row(r, h)) * ld + c * 32 + li;
    };
    if (WAVES == 1) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) out[addr(c, r)] = acc[c][r];
        return;
    }
    const int l = h * 32 + li;
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) lds[((w * NC + c) * 16 + r) * 64 + l] = acc[c][r];
    __syncthreads();
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            if ((r % WAVES) != w) continue;
            float s = 0.f;
#pragma unroll
            for (int ww = 0; ww < WAVES; ++ww) s += lds[((ww * NC + c) * 16 + r) * 64 + l];
            out[addr(c, r)] = s;
        }
}

// A transposed 32-feature accumulator (register = feature acc_row(r, h), lane = row li of the strip) summed over
// the waves and written row-major, rows `ld` floats apart: register group g = r/4 is four consecutive features,
// one 16-byte store per lane; wave g % WAVES writes group g.
template <int WAVES>
__device__ __forceinline__ void reduce_store_rows(const f32x16& acc, float* __restrict__ out, int row0, int w, int li,
                                                  int h, float* __restrict__ lds, size_t ld) {
    const int l = h * 32 + li;
    if (WAVES > 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) lds[(w * 16 + r) * 64 + l] = acc[r];
        __syncthreads();
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        if (WAVES > 1 && (g % WAVES) != w) continue;
        float s[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = 4 * g + j;
            s[j] = acc[r];
            if (WAVES > 1) {
                s[j] = 0.f;
#pragma unroll
                for (int ww = 0; ww < WAVES; ++ww) s[j] += lds[(ww * 16 + r) * 64 + l];
            }
        }
        *reinterpret_cast<f32x4*>(out + (size_t)(row0 + li) * ld + 8 * g + 4 * h) = (f32x4){s[0], s[1], s[2], s[3]};
    }
}

// Like reduce_store (row-major form), but the reduced tile goes to two arrays.
template <int D, int WAVES>
__device__ __forceinline__ void reduce_store2(f32x16 (&acc)[D / 32], float* __restrict__ out, float* __restrict__ out2,
                                              int row0, int w, int li, int h, float* __restrict__ lds) {
    constexpr int NC = D / 32;
    const int l = h * 32 + li;
    if (WAVES > 1) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) lds[((w * NC + c) * 16 + r) * 64 + l] = acc[c][r];
        __syncthreads();
    }
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            if (WAVES > 1 && (r % WAVES) != w) continue;
            float s = acc[c][r];
            if (WAVES > 1) {
                s = 0.f;
#pragma unroll
                for (int ww = 0; ww < WAVES; ++ww) s += lds[((ww * NC + c) * 16 + r) * 64 + l];
            }
            const size_t a = (size_t)(row0 + acc_row(r, h)) * D + c * 32 + li;
            out[a] = s;
            out2[a] = s;
        }
}

}  // namespace spion
