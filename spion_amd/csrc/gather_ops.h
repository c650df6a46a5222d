// Gathers of whole rows for one-wavefront-per-row kernels, without LDS.
//
// A wavefront holds a chunk of up to 64 pattern entries one per lane and fetches the entries' rows (D floats, D = 4 LPR)
// LPR lanes to a row, 16 bytes per lane, G = 64 / LPR rows per load instruction.  Lane l owns entry
// (l % LPR) * G + l / LPR of the chunk, so that the LPR entries group g = l / LPR fetches (entry j*G + g in
// instruction j) are the entries its own LPR lanes own: every exchange stays inside a group of LPR lanes (a
// ds_bpermute for the broadcast of an entry's row and weight, DPP moves for the sums), nothing goes through LDS
// memory, and the number of wavefronts in flight -- what bounds these latency-bound kernels -- is not limited by LDS
// space.  (Staging the gathered rows through a wave-private LDS tile instead made the same kernels three to five
// times slower; the broadcasts as two DPP moves each instead of the permute change nothing: 1.245 against 1.247 ms
// for a step of 20 M entries.)
#pragma once
#include <hip/hip_runtime.h>

namespace spion {

typedef float gather_f32x4 __attribute__((ext_vector_type(4)));

// The rows are fetched with buffer loads: a 32-bit byte offset per lane (row * ld + piece, two VALU instructions)
// instead of a 64-bit address (five), which matters in kernels whose bound is VALU issue.  X: first row of the head
// (wave-uniform); the rows of a head span less than 2 GiB.
typedef __amdgpu_buffer_rsrc_t gather_rsrc_t;
typedef unsigned gather_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ gather_rsrc_t gather_rsrc(const float* X) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(X), 0, 0x7ffffffc, 0x00020000);
}
__device__ __forceinline__ gather_f32x4 gather_load16(gather_rsrc_t r, int row, int ld, int piece) {
    return __builtin_bit_cast(gather_f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (row * ld + 4 * piece) * 4, 0, 0));
}

template <int LPR>
__device__ __forceinline__ int gather_entry_of_lane(int lane) {
    constexpr int G = 64 / LPR;
    return (lane % LPR) * G + lane / LPR;
}

// sum over the LPR lanes of a group (quad swaps, the mirror image of the half row, of the row, then the other row)
template <int LPR>
__device__ __forceinline__ float gather_group_sum(float v) {
    static_assert(LPR == 4 || LPR == 8 || LPR == 16 || LPR == 32, "4 to 32 lanes per row");
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // xor 1
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // xor 2
    if constexpr (LPR >= 8)
        v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // 7 - i
    if constexpr (LPR >= 16)
        v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // 15 - i
    if constexpr (LPR >= 32) v += __shfl_xor(v, 16, 64);
    return v;
}

// Dot products of the rows X[row_l] (row stride ld; row_l: row index of the lane's entry; nk entries in the chunk)
// with the vector whose piece 4*(lane % LPR) .. +3 the lane holds in a4: one result per lane, for the lane's own
// entry.  Only the load instructions that carry entries are issued; lanes whose entry is past nk get 0 or a partial
// value to ignore.
template <int LPR>
__device__ __forceinline__ float gather_dot(const gather_f32x4 a4, const float* __restrict__ X, int ld, int row_l,
                                            int nk, int lane) {
    constexpr int G = 64 / LPR;
    const int base = lane & ~(LPR - 1), cl = lane & (LPR - 1);
    const gather_rsrc_t rx = gather_rsrc(X);
    gather_f32x4 x[LPR];
#pragma unroll
    for (int j = 0; j < LPR; ++j) {
        const int rr = __shfl(row_l, base + j, 64);
        if (j * G < nk) x[j] = gather_load16(rx, rr, ld, cl);
    }
    float r = 0.f;
#pragma unroll
    for (int j = 0; j < LPR; ++j) {
        if (j * G < nk) {
            float sj = x[j].x * a4.x;
            sj = fmaf(x[j].y, a4.y, sj);
            sj = fmaf(x[j].z, a4.z, sj);
            sj = fmaf(x[j].w, a4.w, sj);
            sj = gather_group_sum<LPR>(sj);
            r = cl == j ? sj : r;
        }
    }
    return r;
}

// acc += sum over the chunk's entries (weight w_l and row index row_l of the lane's entry; nk entries) of
// w * X[row][:]; the lane accumulates the piece 4*(lane % LPR) .. +3 of the rows its group fetches.
template <int LPR>
struct GatherRowAcc {
    gather_f32x4 acc;
    __device__ __forceinline__ void clear() { acc = (gather_f32x4){0.f, 0.f, 0.f, 0.f}; }
    __device__ __forceinline__ void chunk(float w_l, int row_l, int nk, const float* __restrict__ X, int ld,
                                          int lane) {
        constexpr int G = 64 / LPR;
        const int base = lane & ~(LPR - 1), cl = lane & (LPR - 1);
        const gather_rsrc_t rx = gather_rsrc(X);
        float w[LPR];
        gather_f32x4 x[LPR];
#pragma unroll
        for (int j = 0; j < LPR; ++j) {
            w[j] = __shfl(w_l, base + j, 64);
            const int rr = __shfl(row_l, base + j, 64);
            if (j * G < nk) x[j] = gather_load16(rx, rr, ld, cl);
        }
#pragma unroll
        for (int j = 0; j < LPR; ++j)
            if (j * G < nk) acc += w[j] * x[j];  // entries past nk inside a carried instruction have weight 0
    }
    // sum over the groups; every lane then holds the four floats 4*(lane % LPR) .. of the result row
    __device__ __forceinline__ gather_f32x4 total() const {
        gather_f32x4 a = acc;
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1)
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] += __shfl_xor(a[e], o, 64);
        return a;
    }
};

}  // namespace spion
