// Hybrid kernels for element-sparse patterns (d = 32): the well-filled aligned 32 x 32 tiles of the pattern (the
// local window of a "window + random columns" pattern, say) run as dense MFMA tiles with a bit mask for the entries
// that are absent, the remaining entries as per-row gathers; the softmax statistics are merged across the two
// parts, and P stays in CSR order exactly as the reference's kernels leave it (models/block_attn_mask.cu:88-140):
// a tile's entries of one row are consecutive in that row's CSR run, so `first position + number of present
// columns to the left` addresses them.
//
// Per pattern entry the gather path costs about as much machine time as 1/80 of a 32 x 32 MFMA tile, so a tile
// with more than ~10 % of its entries present is cheaper dense.
//
// The two parts run as separate launches, each at the occupancy that suits it: the tile kernels (one wavefront per
// strip of 32 rows or columns when strips hold few dense tiles, else a work-group of four wavefronts, wavefront w
// taking the strip's dense tiles w, w+4, ...) and the gather kernels (one wavefront per row or column of the
// remainder, sixteen wavefronts per CU, because the gathers are bound by the number of requests in flight).
// Forward: remainder logits and their row statistics, then the tiles (which merge the statistics and fix the row's
// maximum and denominator), then the remainder's probabilities and share of O.  Backward: tile part then remainder
// part of the row pass, the same for the column pass; the remainder kernels add to what the tile kernels wrote
// (each row or column has exactly one writer per launch).
#pragma once
#include <type_traits>
#include "gather_ops.h"
#include "tile_kernels.h"

namespace spion {

// The analysed pattern as the kernels see it (device pointers, shared by all heads).
struct HybIndex {
    // dense tiles, by block row: tiles t_rp[I] .. t_rp[I+1]-1 of block row I; per tile its block column and, per
    // row of the tile, the position of the row's first entry inside a head's P and the 32-bit set of present columns
    const int* t_rp;
    const int* t_col;
    const int* t_pos;        // [tiles][32]
    const unsigned* t_bits;  // [tiles][32]
    // the same tiles by block column: tile ids t_ct[t_cp[J]] .. of block column J and their block rows t_ci
    const int* t_cp;
    const int* t_ct;
    const int* t_ci;
    // remainder entries in CSR form (r_off [L+1], columns, positions inside a head's P) and in CSC form (c_ptr
    // [L+1], rows ascending within a column, index of the entry in the CSR list); nr entries per head
    const int* r_off;
    const int* r_col;
    const int* r_pos;
    const int* c_ptr;
    const int* c_row;
    const int* c_src;
    int nr;
    int nt;  // dense tiles in all
};

// Tile kernels come in two shapes: one wavefront per strip (strips of up to HYB_MAXT1 dense tiles: the window
// patterns this path is for have about five; the wavefront walks them one after the other, nothing is shared and
// nothing waits at a barrier) and four wavefronts per strip (up to 4 * HYB_MAXT4 dense tiles).  With a handful of
// tiles per strip these launches live on latency, and a strip handled by one wavefront costs a quarter of the
// wavefront start-ups, index look-ups and final reductions.
constexpr int HYB_MAXT1 = 6;    // dense tiles whose logits a single wavefront keeps in registers (forward)
constexpr int HYB_MAXT4 = 4;    // the same per wavefront when four share a strip
constexpr int HYB_MAX_ROW_TILES = 4 * HYB_MAXT4;
constexpr int HYB_GWAVES = 4;    // wavefronts (rows / columns) per work-group of the gather kernels
constexpr float HYB_ABSENT = -1.0e30f;  // logit of an entry that is not in the pattern: exp2 gives exactly 0
// two wavefronts per SIMD, each with the next tile's operands in flight while it works on one
#define SPION_HYB_KERNEL(W) __global__ __launch_bounds__(64 * (W)) __attribute__((amdgpu_waves_per_eu(2, 2)))

// What the tile kernels request ahead of a tile: two operand tiles (raw 16-byte pieces, linear), the tile of P in the
// col-owner layout, and -- one tile further ahead, because the addresses of P come out of it -- the tile's index:
// block column (or row), and position and present-column set of tile row li (lane li and lane 32 + li hold the same).
struct HybPre {
    f32x4 a[4], b[4];
    float p[16];
    float g_l;
    int pos_l, blk;
    unsigned bits_l;
};

__device__ __forceinline__ void hyb_fetch_index(const HybIndex& ix, int t, int li, HybPre& x) {
    x.pos_l = ix.t_pos[(size_t)t * 32 + li];
    x.bits_l = ix.t_bits[(size_t)t * 32 + li];
}

// One value per tile row, held by lane li (and 32 + li) for row li, to the 16 rows acc_row(q, h), q = 0..15, a lane
// works on: through 32 words of the wavefront's own LDS space.
__device__ __forceinline__ void hyb_rows_from_lanes(int* xs, int l, int h, int v, int (&out)[16]) {
    xs[l] = v;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int4 p = *reinterpret_cast<const int4*>(xs + 8 * g + 4 * h);
        out[4 * g + 0] = p.x, out[4 * g + 1] = p.y, out[4 * g + 2] = p.z, out[4 * g + 3] = p.w;
    }
}
__device__ __forceinline__ void hyb_tile_rows(int* xs, int l, int h, const HybPre& x, int (&pos)[16],
                                              unsigned (&bits)[16]) {
    int b[16];
    hyb_rows_from_lanes(xs, l, h, x.pos_l, pos);
    hyb_rows_from_lanes(xs + 64, l, h, (int)x.bits_l, b);
#pragma unroll
    for (int q = 0; q < 16; ++q) bits[q] = (unsigned)b[q];
}
// The tile of P in the col-owner layout (lane li = column of the tile, register q = row acc_row(q, h)); absent
// entries read as 0 (their offset lies past the end of the buffer).  A tile row's entries are consecutive in memory:
// every instruction touches one run per half-wave.
__device__ __forceinline__ void hyb_load_p_cols(rsrc_t rP, const int (&pos)[16], const unsigned (&bits)[16], int li,
                                                float (&pc)[16]) {
    const unsigned below = (1u << li) - 1u;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
        const bool on = (bits[q] >> li) & 1u;
        pc[q] = ld1(rP, on ? 4 * (pos[q] + __popc(bits[q] & below)) : -1, 0);
    }
}
__device__ __forceinline__ void hyb_store_p_cols(float* __restrict__ Ph, const int (&pos)[16],
                                                 const int (&bits)[16], int li, const float (&pc)[16]) {
    const unsigned below = (1u << li) - 1u;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
        const unsigned b = (unsigned)bits[q];
        if ((b >> li) & 1u) Ph[pos[q] + __popc(b & below)] = pc[q];
    }
}

// Sum of the wavefronts' 32 x 32 accumulators (rows acc_row(r, h) of the strip, columns li) times `factor`, in a
// fixed order, to rows of stride ld.  `lds` (WAVES * 1024 floats, unused for one wavefront) may alias tile space no wavefront uses any
// more: the caller has a barrier between that use and this call.
template <int WAVES>
__device__ __forceinline__ void hyb_reduce_store(const f32x16& acc, float factor, float* __restrict__ out, int ld,
                                                 int row0, int w, int li, int h, float* __restrict__ lds) {
    const int l = h * 32 + li;
    if constexpr (WAVES > 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) lds[(w * 16 + r) * 64 + l] = acc[r];
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        if (WAVES > 1 && (r % WAVES) != w) continue;
        float s = acc[r];
        if constexpr (WAVES > 1) {
            s = 0.f;
#pragma unroll
            for (int ww = 0; ww < WAVES; ++ww) s += lds[(ww * 16 + r) * 64 + l];
        }
        s *= factor;
        out[(size_t)(row0 + acc_row(r, h)) * ld + li] = s;
    }
}

// Two-deep software pipeline over n tiles with two register sets: while tile i is computed, the operands and P of
// tile i + 1 are in flight and so is the index of tile i + 2 (requested first, so that waiting for it leaves the
// younger requests outstanding).  Positions past the end are clamped by the callers (valid, redundant requests).
template <class FetchIdx, class FetchData, class Compute>
__device__ __forceinline__ void hyb_pipeline(int n, HybPre& a, HybPre& b, FetchIdx fetch_idx, FetchData fetch_data,
                                             Compute compute) {
    if (n <= 0) return;
    fetch_idx(a, 0);
    fetch_idx(b, 1);
    fetch_data(a, 0);
    int i = 0;
    for (; i + 1 < n; i += 2) {
        fetch_idx(a, i + 2);
        __builtin_amdgcn_sched_barrier(0);
        fetch_data(b, i + 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(a, i);
        __builtin_amdgcn_sched_barrier(0);
        fetch_idx(b, i + 3);
        __builtin_amdgcn_sched_barrier(0);
        fetch_data(a, i + 2);
        __builtin_amdgcn_sched_barrier(0);
        compute(b, i + 1);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (i < n) compute(a, i);
}

// =================================================================================================
// gather helpers (one wavefront per row / column of the remainder)
// =================================================================================================
// The gather primitives (gather_ops.h) with eight lanes to a 32-float row.
__device__ __forceinline__ int hyb_entry_of_lane(int lane) { return gather_entry_of_lane<8>(lane); }

// Start (in floats) and row stride of head bh in a tensor group: contiguous [NB][L][32] heads (ST = false, compile-time
// figures) or [B][H][L][32] views given by a layout.
template <bool ST>
__device__ __forceinline__ void hyb_head(const HeadLayout& y, int H, int bh, int L, size_t& base, int& ld) {
    size_t bytes;
    head_slice<ST, 32>(y, H, bh, L, base, ld, bytes);
}

__device__ __forceinline__ float hyb_gather_dot(const f32x4 a4, const float* __restrict__ X, int ld, int row_l,
                                                int nk, int lane) {
    return gather_dot<8>(a4, X, ld, row_l, nk, lane);
}
typedef GatherRowAcc<8> HybRowAcc;
#define SPION_HYB_GATHER_KERNEL __global__ __launch_bounds__(64 * HYB_GWAVES) __attribute__((amdgpu_waves_per_eu(6, 8)))

// -------------------------------------------------------------------------------------------------
// Forward, step 1: raw logits (log2 domain) of the remainder entries into P, and per row their maximum and the sum
// of their exponentials relative to it: Stats[bh][row] = {m, z} ({HYB_ABSENT, 0} for a row without remainder).
// -------------------------------------------------------------------------------------------------
template <bool MASK, bool ST>
SPION_HYB_GATHER_KERNEL void hyb_rem_logits_kernel(const float* __restrict__ Q, const float* __restrict__ K,
                                                   const float* __restrict__ pen, float* __restrict__ Raw,
                                                   float2* __restrict__ Stats, HybIndex ix, int L, int NB,
                                                   float scale, Layouts ly) {
    const int lane = threadIdx.x & 63, ent = hyb_entry_of_lane(lane);
    const long long wrow = (long long)xcd_remap((int)blockIdx.x, (int)gridDim.x) * HYB_GWAVES + wave_index();
    if (wrow >= (long long)NB * L) return;
    const int bh = (int)(wrow / L), row = (int)(wrow % L);
    const int r0 = ix.r_off[row], rc = ix.r_off[row + 1] - r0;
    size_t ib;
    int ild;
    hyb_head<ST>(ly.in, ly.H, bh, L, ib, ild);
    float* raw = Raw + (size_t)bh * ix.nr + r0;  // this row's logits, in the order of the remainder's CSR list
    const float c2 = scale * LOG2E;
    f32x4 q4 = reinterpret_cast<const f32x4*>(Q + ib + (size_t)row * ild)[lane & 7];
    q4 *= c2;
    // the logits of the first chunks stay in registers; longer rows go back to what they stored in P
    constexpr int KEEP = 2;
    float vk[KEEP];
    float mx = HYB_ABSENT;
    for (int c0 = 0; c0 < rc; c0 += 64) {
        const int k = c0 + ent;
        const int col = k < rc ? ix.r_col[r0 + k] : 0;
        float v = hyb_gather_dot(q4, K + ib, ild, col, min(64, rc - c0), lane);
        if (k < rc) {
            if (MASK) v -= pen[(size_t)bh * L + col] * LOG2E;
            raw[k] = v;
            mx = fmaxf(mx, v);
        } else {
            v = HYB_ABSENT;
        }
#pragma unroll
        for (int c = 0; c < KEEP; ++c)
            if (c0 == 64 * c) vk[c] = v;
    }
    mx = wave_max(mx);
    float z = 0.f;
#pragma unroll
    for (int c = 0; c < KEEP; ++c)
        if (64 * c < rc) z += __builtin_amdgcn_exp2f(vk[c] - mx);
    for (int k = 64 * KEEP + lane; k < rc; k += 64) z += __builtin_amdgcn_exp2f(raw[k] - mx);
    z = wave_sum(z);
    if (lane == 0) Stats[(size_t)bh * L + row] = make_float2(mx, z);
}

// -------------------------------------------------------------------------------------------------
// Forward, step 2: the dense tiles of a strip.  Logits in the log2 domain as in tile_fwd_kernel; the row's
// maximum and denominator take in the remainder's statistics (Stats in: {m, z} of the remainder; out: {row
// maximum, 1 / denominator} for step 3).  Writes the tiles' probabilities to their CSR positions and O = P.V of the
// tile part (step 3 adds the remainder's share).
// -------------------------------------------------------------------------------------------------
template <bool MASK, int WAVES, int MAXT, bool ST>
SPION_HYB_KERNEL(WAVES) void hyb_tile_fwd_kernel(const float* __restrict__ Q, const float* __restrict__ K,
                                          const float* __restrict__ V, const float* __restrict__ pen,
                                          float* __restrict__ P, float* __restrict__ O, float2* __restrict__ Stats,
                                          const int* __restrict__ offs, HybIndex ix, int L, int nbr, int NB, int nnz,
                                          float scale, Layouts ly) {
    constexpr int D = 32, KH = 16;
    __shared__ float lds_m[WAVES][32], lds_z[WAVES][32];
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][64 * TS];  // two 32-row tiles per wavefront
    __shared__ __attribute__((aligned(16))) int lds_x[WAVES][128];
    float* lds = &lds_t[0][0];  // the final reduction reuses the tile space
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, I = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    size_t ib, ob, ibytes, obytes;
    int ild, old_;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, ibytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    const rsrc_t rQ = make_rsrc(Q + ib, ibytes), rK = make_rsrc(K + ib, ibytes), rV = make_rsrc(V + ib, ibytes);
    const rsrc_t rM = make_rsrc(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
    float* Ph = P + (size_t)bh * nnz;
    float* T = lds_t[w];
    float* Tx = T + 32 * TS;
    int* X = lds_x[w];
    const float c2 = scale * LOG2E;
    const int lin = lin_voff(l, ild), tile_bytes = 32 * ild * 4;

    float q[KH];
    ldr_rows<D>(rQ, (li * ild + h * KH) * 4, I * tile_bytes, q);
#pragma unroll
    for (int s = 0; s < KH; ++s) q[s] *= c2;
    const float2 rem = Stats[(size_t)bh * L + I * 32 + li];  // the remainder of row li

    // ---- index of this wavefront's tiles (positions past the end repeat the last one: valid, redundant) -----
    const int t0 = ix.t_rp[I], cnt = ix.t_rp[I + 1] - t0;
    const int nu = cnt > w ? (cnt - w + WAVES - 1) / WAVES : 0;
    int Js[MAXT], pos_l[MAXT];
    unsigned bits_l[MAXT];  // present columns / first position of tile row li
#pragma unroll
    for (int u = 0; u < MAXT; ++u) {
        const int t = min(t0 + w + min(u, max(nu, 1) - 1) * WAVES, ix.nt - 1);
        Js[u] = ix.t_col[t];
        pos_l[u] = ix.t_pos[(size_t)t * 32 + li];
        bits_l[u] = ix.t_bits[(size_t)t * 32 + li];
    }

    // ---- logits of the tiles, own maximum; the next tile of K is in flight while one is worked on --------
    float m = MASK ? 0.f : -100.f * LOG2E, z = 0.f;
    f32x16 S[MAXT];
    f32x4 raw[2][4];
    float pj[2][16];
    ldr_tile_lin(rK, lin, Js[0] * tile_bytes, ild, raw[0]);
    if constexpr (MASK) ldr_4x4(rM, 16 * h, Js[0] * 128, pj[0]);
#pragma unroll
    for (int u = 0; u < MAXT; ++u) {
        if (u + 1 < MAXT) {
            ldr_tile_lin(rK, lin, Js[u + 1] * tile_bytes, ild, raw[(u + 1) & 1]);
            if constexpr (MASK) ldr_4x4(rM, 16 * h, Js[u + 1] * 128, pj[(u + 1) & 1]);
        } else {
            ldr_tile_lin(rV, lin, Js[0] * tile_bytes, ild, raw[(u + 1) & 1]);  // first tile of V for the last step
        }
        __builtin_amdgcn_sched_barrier(0);
        if (u < nu) {
            f32x16 init = splat16(0.f);
            if constexpr (MASK) {
#pragma unroll
                for (int r = 0; r < 16; ++r) init[r] = -LOG2E * pj[u & 1][r];
            }
            lds_put_lin(Tx, l, raw[u & 1]);
            float kf[KH];
            lds_get_feat32(Tx, li, h, kf);
            S[u] = mma_feat_init<D>(kf, q, init);  // register = key acc_row(r, h), lane = query li
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (!((bits_l[u] >> acc_row(r, h)) & 1u)) S[u][r] = HYB_ABSENT;
            m = max16(S[u], m);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    m = fmaxf(m, __shfl_xor(m, 32, 64));
#pragma unroll
    for (int u = 0; u < MAXT; ++u) {
        if (u < nu) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float e = __builtin_amdgcn_exp2f(S[u][r] - m);
                S[u][r] = e;
                z += e;
            }
        }
    }
    const float m_own = m;
    z += __shfl_xor(z, 32, 64);

    // ---- merge: row maximum and denominator over the tiles of all wavefronts and the remainder ----
    float Mx = fmaxf(rem.x, m);
    float Z = rem.y * __builtin_amdgcn_exp2f(rem.x - Mx);
    if constexpr (WAVES > 1) {
        if (h == 0) {
            lds_m[w][li] = m;
            lds_z[w][li] = z;
        }
        __syncthreads();
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) Mx = fmaxf(Mx, lds_m[ww][li]);
        Z = rem.y * __builtin_amdgcn_exp2f(rem.x - Mx);
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) Z += lds_z[ww][li] * __builtin_amdgcn_exp2f(lds_m[ww][li] - Mx);
    } else {
        Z += z * __builtin_amdgcn_exp2f(m - Mx);
    }
    {
        const int row = I * 32 + li;
        const int n_i = offs[row + 1] - offs[row];
        Z += (float)(L - n_i) * __builtin_amdgcn_exp2f(-Mx);
    }
    const float zinv = 1.0f / Z;  // +inf denominator -> 0 -> P = 0, as in the reference
    const float rinv = __builtin_amdgcn_exp2f(m_own - Mx) * zinv;

    // ---- probabilities, O += P.V, P to its CSR positions; V of the next tile in flight ------------------
    f32x16 o[1] = {splat16(0.f)};
#pragma unroll
    for (int u = 0; u < MAXT; ++u) {
        constexpr int FIRST = MAXT & 1;  // the set the first tile of V went to
        if (u + 1 < MAXT) ldr_tile_lin(rV, lin, Js[u + 1] * tile_bytes, ild, raw[(FIRST + u + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
        if (u < nu) {
            lds_put_lin(Tx, l, raw[(FIRST + u) & 1]);
            float p[16], vb[1][16], pc[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) p[r] = S[u][r] * rinv;
            lds_put_rows(T, li, h, p);
            lds_get_cols(Tx, li, h, vb[0]);
            lds_get_cols(T, li, h, pc);
            mma_b<D>(p, vb, o);
            int pos[16], bits[16];
            hyb_rows_from_lanes(X, l, h, pos_l[u], pos);
            hyb_rows_from_lanes(X + 64, l, h, (int)bits_l[u], bits);
            hyb_store_p_cols(Ph, pos, bits, li, pc);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (WAVES > 1) __syncthreads();
    // every wavefront has consumed the remainder's statistics by now: replace them by the row's final ones
    if (w == 0 && h == 0) Stats[(size_t)bh * L + I * 32 + li] = make_float2(Mx, zinv);
    hyb_reduce_store<WAVES>(o[0], 1.0f, O + ob, old_, I * 32, w, li, h, lds);
}

// -------------------------------------------------------------------------------------------------
// Forward, step 3: probabilities of the remainder entries from their raw logits and the row's {maximum,
// 1 / denominator}; their share of O is added to what step 2 wrote.  Ocache (optional): second copy of O.
// -------------------------------------------------------------------------------------------------
template <bool ST>
SPION_HYB_GATHER_KERNEL void hyb_rem_pv_kernel(const float* __restrict__ V, const float* __restrict__ Raw,
                                               float* __restrict__ P, float* __restrict__ O,
                                               float* __restrict__ Ocache,
                                               const float2* __restrict__ Stats, HybIndex ix, int L, int NB, int nnz,
                                               Layouts ly) {
    const int lane = threadIdx.x & 63, ent = hyb_entry_of_lane(lane);
    const long long wrow = (long long)xcd_remap((int)blockIdx.x, (int)gridDim.x) * HYB_GWAVES + wave_index();
    if (wrow >= (long long)NB * L) return;
    const int bh = (int)(wrow / L), row = (int)(wrow % L);
    const int r0 = ix.r_off[row], rc = ix.r_off[row + 1] - r0;
    size_t ib, ob;
    int ild, old_;
    hyb_head<ST>(ly.in, ly.H, bh, L, ib, ild);
    hyb_head<ST>(ly.out, ly.H, bh, L, ob, old_);
    float* Ph = P + (size_t)bh * nnz;
    const float* raw = Raw + (size_t)bh * ix.nr + r0;
    const float2 st = Stats[(size_t)bh * L + row];
    HybRowAcc acc;
    acc.clear();
    for (int c0 = 0; c0 < rc; c0 += 64) {
        const int k = c0 + ent;
        float wgt = 0.f;
        int col = 0;
        if (k < rc) {
            const int pp = ix.r_pos[r0 + k];
            wgt = __builtin_amdgcn_exp2f(raw[k] - st.x) * st.y;
            col = ix.r_col[r0 + k];
            __builtin_nontemporal_store(wgt, Ph + pp);  // written once, not read again before the backward
        }
        acc.chunk(wgt, col, min(64, rc - c0), V + ib, ild, lane);
    }
    const f32x4 tot = acc.total();
    if (lane < 8) {
        f32x4* orow = reinterpret_cast<f32x4*>(O + ob + (size_t)row * old_) + lane;
        const f32x4 sum = *orow + tot;
        *orow = sum;
        if (Ocache) reinterpret_cast<f32x4*>(Ocache + ((size_t)bh * L + row) * 32)[lane] = sum;  // own copy: contiguous
    }
}

// -------------------------------------------------------------------------------------------------
// Backward, row pass, dense tiles: g_i = dO_i . O_i (G receives -g for the other kernels); dP^T - g = V_J.dO_I^T
// chain started from -g, dS' = (dP - g)*P, dQ = sum dS'.K_J / sqrt(d).
// -------------------------------------------------------------------------------------------------
template <int WAVES, bool ST>
SPION_HYB_KERNEL(WAVES) void hyb_tile_bwd_row_kernel(const float* __restrict__ K, const float* __restrict__ V,
                                              const float* __restrict__ P, const float* __restrict__ dO,
                                              const float* __restrict__ Out, float* __restrict__ G,
                                              float* __restrict__ dQ, HybIndex ix, int L, int nbr, int NB, int nnz,
                                              float scale, Layouts ly) {
    constexpr int D = 32, KH = 16;
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][64 * TS];
    __shared__ __attribute__((aligned(16))) int lds_x[WAVES][128];
    float* lds = &lds_t[0][0];
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, I = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    size_t ib, ob, gb, ibytes, obytes, gbytes;
    int ild, old_, gld;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, ibytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    head_slice<ST, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rK = make_rsrc(K + ib, ibytes), rV = make_rsrc(V + ib, ibytes);
    const rsrc_t rdO = make_rsrc(dO + ob, obytes), rO = make_rsrc(Out + ob, obytes);
    const rsrc_t rP = make_rsrc(P + (size_t)bh * nnz, (size_t)nnz * 4);
    float* T = lds_t[w];
    float* Tx = T + 32 * TS;
    int* X = lds_x[w];
    const int lin = lin_voff(l, ild), tile_bytes = 32 * ild * 4;

    float go[KH], oo[KH];
    ldr_rows<D>(rdO, (li * old_ + h * KH) * 4, I * 32 * old_ * 4, go);
    ldr_rows<D>(rO, (li * old_ + h * KH) * 4, I * 32 * old_ * 4, oo);
    float g = 0.f;
#pragma unroll
    for (int s = 0; s < KH; ++s) g = fmaf(go[s], oo[s], g);
    g += __shfl_xor(g, 32, 64);
    if (w == 0 && h == 0) G[(size_t)bh * L + I * 32 + li] = -g;
    const f32x16 gneg = splat16(-g);

    const int t0 = ix.t_rp[I], cnt = ix.t_rp[I + 1] - t0;
    const int n = cnt > w ? (cnt - w + WAVES - 1) / WAVES : 0;
    f32x16 acc[1] = {splat16(0.f)};
    HybPre xa, xb;
    hyb_pipeline(
        n, xa, xb,
        [&](HybPre& x, int i) {
            const int t = t0 + w + min(i, n - 1) * WAVES;
            x.blk = ix.t_col[t];
            hyb_fetch_index(ix, t, li, x);
        },
        [&](HybPre& x, int) {
            int pos[16];
            unsigned bits[16];
            hyb_tile_rows(X, l, h, x, pos, bits);
            ldr_tile_lin(rV, lin, x.blk * tile_bytes, ild, x.a);
            hyb_load_p_cols(rP, pos, bits, li, x.p);
            ldr_tile_lin(rK, lin, x.blk * tile_bytes, ild, x.b);
        },
        [&](HybPre& x, int) {
            float pr[16], vt[KH], kb[1][16];
            lds_put_lin(Tx, l, x.a);
            lds_get_feat32(Tx, li, h, vt);
            lds_put_cols(T, li, h, x.p);
            lds_get_rows(T, li, h, pr);                        // pr[r] = P[query li][key acc_row(r, h)]
            const f32x16 dp = mma_feat_init<D>(vt, go, gneg);  // dp[r] = dO_i . v_j - g_i
            lds_put_lin(Tx, l, x.b);
            lds_get_cols(Tx, li, h, kb[0]);
            float ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = dp[r] * pr[r];
            mma_b<D>(ds, kb, acc);
        });
    if constexpr (WAVES > 1) __syncthreads();
    hyb_reduce_store<WAVES>(acc[0], scale, dQ + gb, gld, I * 32, w, li, h, lds);
}

// -------------------------------------------------------------------------------------------------
// Backward, row pass, remainder: dS = (dO_i . v_j - g_i) * P / sqrt(d), dQ_i += sum dS . K[col].  The column pass
// walks the same entries column after column; looking P and dS up there inside a head's full P and dS (two arrays
// of nnz floats, more than the L2 cache holds per head) would fetch a memory sector for every four bytes, so this
// kernel leaves the pairs {dS, P} of the remainder alone in one compact list (Pairs [NB][nr], row order, inside the
// caller's dS scratch), small enough per head for the column pass to find in the L2 cache.
// -------------------------------------------------------------------------------------------------
template <bool ST>
SPION_HYB_GATHER_KERNEL void hyb_rem_bwd_row_kernel(const float* __restrict__ K, const float* __restrict__ V,
                                                    const float* __restrict__ P, const float* __restrict__ dO,
                                                    const float* __restrict__ G, float2* __restrict__ Pairs,
                                                    float* __restrict__ dQ, HybIndex ix, int L, int NB, int nnz,
                                                    float scale, Layouts ly) {
    const int lane = threadIdx.x & 63, ent = hyb_entry_of_lane(lane);
    const long long wrow = (long long)xcd_remap((int)blockIdx.x, (int)gridDim.x) * HYB_GWAVES + wave_index();
    if (wrow >= (long long)NB * L) return;
    const int bh = (int)(wrow / L), row = (int)(wrow % L);
    const int r0 = ix.r_off[row], rc = ix.r_off[row + 1] - r0;
    if (rc == 0) return;
    size_t ib, ob, gb;
    int ild, old_, gld;
    hyb_head<ST>(ly.in, ly.H, bh, L, ib, ild);
    hyb_head<ST>(ly.out, ly.H, bh, L, ob, old_);
    hyb_head<ST>(ly.grad, ly.H, bh, L, gb, gld);
    const f32x4 go4 = reinterpret_cast<const f32x4*>(dO + ob + (size_t)row * old_)[lane & 7];
    const float* Ph = P + (size_t)bh * nnz;
    float2* pairs = Pairs + (size_t)bh * ix.nr;
    const float gneg = G[(size_t)bh * L + row];
    HybRowAcc acc;
    acc.clear();
    for (int c0 = 0; c0 < rc; c0 += 64) {
        const int k = c0 + ent;
        const int col = k < rc ? ix.r_col[r0 + k] : 0;
        const int pp = k < rc ? ix.r_pos[r0 + k] : 0;
        const float pv = k < rc ? Ph[pp] : 0.f;
        const int nk = min(64, rc - c0);
        const float dp = hyb_gather_dot(go4, V + ib, ild, col, nk, lane);
        float dsv = 0.f;
        if (k < rc) {
            dsv = (dp + gneg) * pv * scale;
            pairs[r0 + k] = make_float2(dsv, pv);
        }
        acc.chunk(dsv, col, nk, K + ib, ild, lane);
    }
    const f32x4 tot = acc.total();
    if (lane < 8) {
        f32x4* qrow = reinterpret_cast<f32x4*>(dQ + gb + (size_t)row * gld) + lane;
        *qrow = *qrow + tot;
    }
}

// -------------------------------------------------------------------------------------------------
// Backward, column pass, dense tiles: dK_J = sum_I dS_IJ^T Q_I / sqrt(d), dV_J = sum_I P_IJ^T dO_I; dP - g is
// recomputed per tile by a chain started from the stored -g.
// -------------------------------------------------------------------------------------------------
template <int WAVES, bool ST>
SPION_HYB_KERNEL(WAVES) void hyb_tile_bwd_col_kernel(const float* __restrict__ Q, const float* __restrict__ V,
                                              const float* __restrict__ P, const float* __restrict__ dO,
                                              const float* __restrict__ G, float* __restrict__ dK,
                                              float* __restrict__ dV, HybIndex ix, int L, int nbr, int NB, int nnz,
                                              float scale, Layouts ly) {
    constexpr int D = 32, KH = 16;
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][64 * TS];
    __shared__ __attribute__((aligned(16))) int lds_x[WAVES][128];
    float* lds = &lds_t[0][0];
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, J = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    size_t ib, ob, gb, ibytes, obytes, gbytes;
    int ild, old_, gld;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, ibytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    head_slice<ST, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rQ = make_rsrc(Q + ib, ibytes), rV = make_rsrc(V + ib, ibytes);
    const rsrc_t rdO = make_rsrc(dO + ob, obytes);
    const rsrc_t rG = make_rsrc(G + (size_t)bh * L, (size_t)L * 4);
    const rsrc_t rP = make_rsrc(P + (size_t)bh * nnz, (size_t)nnz * 4);
    float* Tq = lds_t[w];
    float* To = Tq + 32 * TS;
    int* X = lds_x[w];
    const int lin_i = lin_voff(l, ild), lin_o = lin_voff(l, old_);

    float vt[KH];
    ldr_rows<D>(rV, (li * ild + h * KH) * 4, J * 32 * ild * 4, vt);

    f32x16 ak[1] = {splat16(0.f)}, av[1] = {splat16(0.f)};
    const int e0 = ix.t_cp[J], ecnt = ix.t_cp[J + 1] - e0;
    const int n = ecnt > w ? (ecnt - w + WAVES - 1) / WAVES : 0;
    HybPre xa, xb;
    hyb_pipeline(
        n, xa, xb,
        [&](HybPre& x, int i) {
            const int e = e0 + w + min(i, n - 1) * WAVES;
            x.blk = ix.t_ci[e];
            hyb_fetch_index(ix, ix.t_ct[e], li, x);
        },
        [&](HybPre& x, int) {
            int pos[16];
            unsigned bits[16];
            hyb_tile_rows(X, l, h, x, pos, bits);
            ldr_tile_lin(rQ, lin_i, x.blk * 32 * ild * 4, ild, x.a);
            ldr_tile_lin(rdO, lin_o, x.blk * 32 * old_ * 4, old_, x.b);
            hyb_load_p_cols(rP, pos, bits, li, x.p);  // p[r] = P[query acc_row(r, h)][key li]
            x.g_l = ld1(rG, li * 4, x.blk * 128);
        },
        [&](HybPre& x, int) {
            float go[KH], qb[1][16], ob[1][16];
            int gn[16];
            lds_put_lin(Tq, l, x.a);
            lds_put_lin(To, l, x.b);
            hyb_rows_from_lanes(X, l, h, __builtin_bit_cast(int, x.g_l), gn);
            lds_get_feat32(To, li, h, go);
            lds_get_cols(Tq, li, h, qb[0]);
            lds_get_cols(To, li, h, ob[0]);
            f32x16 init;
#pragma unroll
            for (int r = 0; r < 16; ++r) init[r] = __builtin_bit_cast(float, gn[r]);
            const f32x16 dp = mma_feat_init<D>(go, vt, init);  // dO_i . v_j - g_i, i = acc_row(r, h), j = li
            float ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = dp[r] * x.p[r];
            mma_b<D>(ds, qb, ak);
            mma_b<D>(x.p, ob, av);
        });
    if constexpr (WAVES > 1) __syncthreads();
    hyb_reduce_store<WAVES>(ak[0], scale, dK + gb, gld, J * 32, w, li, h, lds);
    if constexpr (WAVES > 1) __syncthreads();
    hyb_reduce_store<WAVES>(av[0], 1.0f, dV + gb, gld, J * 32, w, li, h, lds);
}

// -------------------------------------------------------------------------------------------------
// Backward, column pass, remainder: dK_j += sum_i dS_ij Q_i, dV_j += sum_i P_ij dO_i over the remainder's
// transposed index, from the compact {dS, P} pairs of the row pass (dS already carries the 1/sqrt(d)).
// -------------------------------------------------------------------------------------------------
template <bool ST>
__global__ __launch_bounds__(64 * HYB_GWAVES) void hyb_rem_bwd_col_kernel(  // two gathers in flight per entry: four waves per SIMD
    const float* __restrict__ Q, const float* __restrict__ dO,
                                                    const float2* __restrict__ Pairs,
                                                    float* __restrict__ dK, float* __restrict__ dV, HybIndex ix, int L,
                                                    int NB, Layouts ly) {
    const int lane = threadIdx.x & 63, ent = hyb_entry_of_lane(lane);
    const long long wcol = (long long)xcd_remap((int)blockIdx.x, (int)gridDim.x) * HYB_GWAVES + wave_index();
    if (wcol >= (long long)NB * L) return;
    const int bh = (int)(wcol / L), colj = (int)(wcol % L);
    const int c0p = ix.c_ptr[colj], cnt = ix.c_ptr[colj + 1] - c0p;
    if (cnt == 0) return;
    size_t ib, ob, gb;
    int ild, old_, gld;
    hyb_head<ST>(ly.in, ly.H, bh, L, ib, ild);
    hyb_head<ST>(ly.out, ly.H, bh, L, ob, old_);
    hyb_head<ST>(ly.grad, ly.H, bh, L, gb, gld);
    const float2* pairs = Pairs + (size_t)bh * ix.nr;
    HybRowAcc ak, av;
    ak.clear();
    av.clear();
    for (int c0 = 0; c0 < cnt; c0 += 64) {
        const int e = c0 + ent;
        float wk = 0.f, wv = 0.f;
        int row = 0;
        if (e < cnt) {
            row = ix.c_row[c0p + e];
            const float2 pr = pairs[ix.c_src[c0p + e]];
            wk = pr.x;
            wv = pr.y;
        }
        const int nk = min(64, cnt - c0);
        ak.chunk(wk, row, nk, Q + ib, ild, lane);
        av.chunk(wv, row, nk, dO + ob, old_, lane);
    }
    const f32x4 tk = ak.total(), tv = av.total();
    if (lane < 8) {
        f32x4* kr = reinterpret_cast<f32x4*>(dK + gb + (size_t)colj * gld) + lane;
        f32x4* vr = reinterpret_cast<f32x4*>(dV + gb + (size_t)colj * gld) + lane;
        *kr = *kr + tk;
        *vr = *vr + tv;
    }
}

// -------------------------------------------------------------------------------------------------
// The same pass with the gathered operands in LDS instead of L2.  A work-group of sixteen wavefronts owns 128 * NC
// columns of a head and walks the sequence in ranges of HYB_CL_ROWS rows, whose Q and dO rows (128 KB) it loads
// once per range.  A group of eight lanes owns NC columns (lane s holds floats 4s .. 4s+3 of their dK and dV rows,
// 8 * NC accumulator registers that live across the ranges) and walks each column's entries -- rows ascending, so the
// entries of a range are the next ones of the column's list -- eight at a time: lane s fetches the s-th entry's row
// and {dS, P} pair with full-width loads, the eight are handed round the group, and every lane adds its 16-byte
// pieces of the Q and dO rows, read from LDS, to its sums.  Each lane's sums run in a fixed order along the column's
// list, so the result does not depend on the launch.
// -------------------------------------------------------------------------------------------------
constexpr int HYB_CL_ROWS = 512, HYB_CL_THREADS = 1024;  // a work-group owns NC * 128 columns: 1024 (NC = 8) or 512
// x of another lane of the same row of sixteen: quad_perm (CTRL = 0x55 * k: lane k of the own quad) or row_half_mirror
// (0x141: lane 7 - i of the own eight)
template <int CTRL>
__device__ __forceinline__ int hyb_dpp(int x) {
    return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xf, 0xf, false);
}
// The list of a column: entries c_ptr[j] .. c_ptr[j+1]-1, their rows c_row (ascending) and c_src, the index of the
// entry's weights -- PAIRS: in the compact {dS, P} list of a head ([NB][n] float2; the sums are added to what the tile
// part left in dK and dV); otherwise in the head's dS and P arrays ([NB][n] floats each; the sums are the result).
template <bool ST, bool PAIRS, int NC>
__global__ __launch_bounds__(HYB_CL_THREADS) void hyb_rem_bwd_col_lds_kernel(
    const float* __restrict__ Q, const float* __restrict__ dO, const float2* __restrict__ Pairs,
    const float* __restrict__ dSa, const float* __restrict__ Pa, float* __restrict__ dK, float* __restrict__ dV,
    const int* __restrict__ c_ptr, const int* __restrict__ c_row, const int* __restrict__ c_src, int n, int L, int NB,
    Layouts ly) {
    __shared__ f32x4 sq[HYB_CL_ROWS * 8], so[HYB_CL_ROWS * 8];
    constexpr int HYB_CL_COLS = NC * (HYB_CL_THREADS / 8);
    const int ncg = L / HYB_CL_COLS;
    const int item = xcd_remap((int)blockIdx.x, (int)gridDim.x);  // the work-groups of a head share an XCD's L2
    const int bh = item / ncg, cg = item % ncg;
    const int t = threadIdx.x, grp = t >> 3, sub = t & 7, lane = t & 63;
    size_t ib, ob, gb;
    int ild, old_, gld;
    hyb_head<ST>(ly.in, ly.H, bh, L, ib, ild);
    hyb_head<ST>(ly.out, ly.H, bh, L, ob, old_);
    hyb_head<ST>(ly.grad, ly.H, bh, L, gb, gld);
    const float2* pairs = PAIRS ? Pairs + (size_t)bh * n : nullptr;
    const float* dsh = PAIRS ? nullptr : dSa + (size_t)bh * n;
    const float* ph = PAIRS ? nullptr : Pa + (size_t)bh * n;
    auto weights = [&](int src) { return PAIRS ? pairs[src] : (float2){dsh[src], ph[src]}; };
    f32x4 ak[NC], av[NC];
    int e[NC], eend[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int col = cg * HYB_CL_COLS + c * (HYB_CL_THREADS / 8) + grp;
        ak[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
        av[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
        e[c] = c_ptr[col];
        eend[c] = c_ptr[col + 1];
    }
    for (int r0 = 0; r0 < L; r0 += HYB_CL_ROWS) {
        __syncthreads();  // everybody has finished with the previous range
#pragma unroll
        for (int k = 0; k < HYB_CL_ROWS * 8 / HYB_CL_THREADS; ++k) {
            const int idx = t + k * HYB_CL_THREADS, row = r0 + (idx >> 3), piece = idx & 7;
            sq[idx] = reinterpret_cast<const f32x4*>(Q + ib + (size_t)row * ild)[piece];
            so[idx] = reinterpret_cast<const f32x4*>(dO + ob + (size_t)row * old_)[piece];
        }
        __syncthreads();
        const int rend = r0 + HYB_CL_ROWS;
        auto fetch_idx = [&](int c, int& row, int& src) {
            const int my = e[c] + sub;
            const bool ok = my < eend[c];
            row = ok ? c_row[my] : 0x7fffffff;
            src = ok ? c_src[my] : 0;
        };
        // The eight entries go round the group by DPP moves: a quad broadcast hands entry k of a lane's own quad to
        // its four lanes, and the same on the values mirrored within the eight lanes hands over the other quad's
        // entries -- every lane sees all eight, each quad in an order of its own, which is fixed.
        auto add_batch = [&](int c, int lrow, float2 pr) {
            const int wx = __float_as_int(pr.x), wy = __float_as_int(pr.y);
            const int mrow = hyb_dpp<0x141>(lrow), mx = hyb_dpp<0x141>(wx), my_ = hyb_dpp<0x141>(wy);
#define SPION_HYB_ENTRY(CTRL, R, X, Y)                                           \
    {                                                                            \
        const int rk = hyb_dpp<CTRL>(R);                                         \
        const float wk = __int_as_float(hyb_dpp<CTRL>(X)), wv = __int_as_float(hyb_dpp<CTRL>(Y)); \
        ak[c] += sq[rk * 8 + sub] * wk;                                          \
        av[c] += so[rk * 8 + sub] * wv;                                          \
    }
            SPION_HYB_ENTRY(0x00, lrow, wx, wy)
            SPION_HYB_ENTRY(0x55, lrow, wx, wy)
            SPION_HYB_ENTRY(0xaa, lrow, wx, wy)
            SPION_HYB_ENTRY(0xff, lrow, wx, wy)
            SPION_HYB_ENTRY(0x00, mrow, mx, my_)
            SPION_HYB_ENTRY(0x55, mrow, mx, my_)
            SPION_HYB_ENTRY(0xaa, mrow, mx, my_)
            SPION_HYB_ENTRY(0xff, mrow, mx, my_)
#undef SPION_HYB_ENTRY
        };
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            int nn = 8;
            while (nn == 8) {
                int r1, s1;
                fetch_idx(c, r1, s1);
                const bool in = r1 < rend;
                nn = __popcll((__ballot(in) >> (lane & 56)) & 0xffull);
                if (nn == 0) break;
                add_batch(c, in ? r1 - r0 : 0, in ? weights(s1) : (float2){0.f, 0.f});
                e[c] += nn;
            }
        }
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int col = cg * HYB_CL_COLS + c * (HYB_CL_THREADS / 8) + grp;
        f32x4* kr = reinterpret_cast<f32x4*>(dK + gb + (size_t)col * gld) + sub;
        f32x4* vr = reinterpret_cast<f32x4*>(dV + gb + (size_t)col * gld) + sub;
        if constexpr (PAIRS) {
            if (eend[c] == c_ptr[col]) continue;  // a column without remainder entries
            *kr = *kr + ak[c];
            *vr = *vr + av[c];
        } else {
            *kr = ak[c];
            *vr = av[c];
        }
    }
}

// -------------------------------------------------------------------------------------------------
// Forward, step 1, with the K rows in LDS: a work-group of sixteen wavefronts owns 128 * NR query rows of a head and
// walks the keys in ranges of HYB_LL_KEYS, whose K rows (128 KB; with a key mask their penalties too) it loads once
// per range.  A group of eight lanes owns NR rows (their scaled Q rows -- lane i of either quad holds pieces i and
// i + 4 -- and their running {maximum, sum}) and walks each row's remainder entries eight at a time, lane s fetching
// the s-th entry's column; then either quad of the group takes the four entries its own lanes hold, one after the
// other: the column goes round the quad by a DPP move, every lane multiplies its two pieces of the K row, read from
// LDS, two DPP additions make the dot product, and the lane that holds the entry keeps it.  The eight logits are
// stored, and the row's statistics follow batch by batch (maximum raised, sum rescaled).
// -------------------------------------------------------------------------------------------------
constexpr int HYB_LL_KEYS = 1024, HYB_LL_THREADS = 1024;
template <bool MASK, bool ST, int NR>
__global__ __launch_bounds__(HYB_LL_THREADS) void hyb_rem_logits_lds_kernel(
    const float* __restrict__ Q, const float* __restrict__ K, const float* __restrict__ pen, float* __restrict__ Raw,
    float2* __restrict__ Stats, HybIndex ix, int L, int NB, float scale, Layouts ly) {
    __shared__ f32x4 sk[HYB_LL_KEYS * 8];
    __shared__ float spen[MASK ? HYB_LL_KEYS : 1];
    constexpr int ROWS = NR * (HYB_LL_THREADS / 8);
    const int nrg = L / ROWS;
    const int item = xcd_remap((int)blockIdx.x, (int)gridDim.x);  // the work-groups of a head share an XCD's L2
    const int bh = item / nrg, rg = item % nrg;
    const int t = threadIdx.x, grp = t >> 3, sub = t & 7, qi = t & 3, lane = t & 63;
    size_t ib;
    int ild;
    hyb_head<ST>(ly.in, ly.H, bh, L, ib, ild);
    float* raw = Raw + (size_t)bh * ix.nr;
    const float c2 = scale * LOG2E;
    f32x4 q0[NR], q1[NR];
    float m[NR], z[NR];
    int e[NR], eend[NR];
#pragma unroll
    for (int c = 0; c < NR; ++c) {
        const int row = rg * ROWS + c * (HYB_LL_THREADS / 8) + grp;
        const f32x4* qr = reinterpret_cast<const f32x4*>(Q + ib + (size_t)row * ild);
        q0[c] = qr[qi] * c2;
        q1[c] = qr[4 + qi] * c2;
        m[c] = HYB_ABSENT;
        z[c] = 0.f;
        e[c] = ix.r_off[row];
        eend[c] = ix.r_off[row + 1];
    }
    auto fdpp = [](auto ctrl, float x) {
        return __int_as_float(hyb_dpp<decltype(ctrl)::value>(__float_as_int(x)));
    };
    for (int k0 = 0; k0 < L; k0 += HYB_LL_KEYS) {
        __syncthreads();  // everybody has finished with the previous range
#pragma unroll
        for (int k = 0; k < HYB_LL_KEYS * 8 / HYB_LL_THREADS; ++k) {
            const int idx = t + k * HYB_LL_THREADS;
            sk[idx] = reinterpret_cast<const f32x4*>(K + ib + (size_t)(k0 + (idx >> 3)) * ild)[idx & 7];
        }
        if constexpr (MASK) spen[t] = pen[(size_t)bh * L + k0 + t] * LOG2E;
        __syncthreads();
        const int kend = k0 + HYB_LL_KEYS;
#pragma unroll
        for (int c = 0; c < NR; ++c) {
            int nn = 8;
            while (nn == 8) {
                const int my = e[c] + sub;
                const int col = my < eend[c] ? ix.r_col[my] : 0x7fffffff;
                const bool in = col < kend;
                // columns ascend along the list: the entries of this range among the eight are the first nn
                nn = __popcll((__ballot(in) >> (lane & 56)) & 0xffull);
                if (nn == 0) break;
                const int lcol = in ? col - k0 : 0;
                float v = 0.f;
#define SPION_HYB_QUAD_STEP(KQ)                                                                       \
    {                                                                                                 \
        const int ck = hyb_dpp<0x55 * KQ>(lcol);                                                      \
        const f32x4 a0 = sk[ck * 8 + qi], a1 = sk[ck * 8 + 4 + qi];                                   \
        float d = a0.x * q0[c].x;                                                                     \
        d = fmaf(a0.y, q0[c].y, d);                                                                   \
        d = fmaf(a0.z, q0[c].z, d);                                                                   \
        d = fmaf(a0.w, q0[c].w, d);                                                                   \
        d = fmaf(a1.x, q1[c].x, d);                                                                   \
        d = fmaf(a1.y, q1[c].y, d);                                                                   \
        d = fmaf(a1.z, q1[c].z, d);                                                                   \
        d = fmaf(a1.w, q1[c].w, d);                                                                   \
        d += fdpp(std::integral_constant<int, 0xB1>{}, d);                                            \
        d += fdpp(std::integral_constant<int, 0x4E>{}, d);                                            \
        if constexpr (MASK) d -= spen[ck];                                                            \
        v = qi == KQ ? d : v;                                                                         \
    }
                SPION_HYB_QUAD_STEP(0)
                SPION_HYB_QUAD_STEP(1)
                SPION_HYB_QUAD_STEP(2)
                SPION_HYB_QUAD_STEP(3)
#undef SPION_HYB_QUAD_STEP
                if (in) raw[my] = v;
                else v = HYB_ABSENT;
                float bm = v;
                bm = fmaxf(bm, fdpp(std::integral_constant<int, 0xB1>{}, bm));
                bm = fmaxf(bm, fdpp(std::integral_constant<int, 0x4E>{}, bm));
                bm = fmaxf(bm, fdpp(std::integral_constant<int, 0x141>{}, bm));
                const float mnew = fmaxf(m[c], bm);
                float ex = __builtin_amdgcn_exp2f(v - mnew);  // an absent entry gives exactly 0
                ex += fdpp(std::integral_constant<int, 0xB1>{}, ex);
                ex += fdpp(std::integral_constant<int, 0x4E>{}, ex);
                ex += fdpp(std::integral_constant<int, 0x141>{}, ex);
                z[c] = z[c] * __builtin_amdgcn_exp2f(m[c] - mnew) + ex;
                m[c] = mnew;
                e[c] += nn;
            }
        }
    }
#pragma unroll
    for (int c = 0; c < NR; ++c) {
        const int row = rg * ROWS + c * (HYB_LL_THREADS / 8) + grp;
        if (sub == 0) Stats[(size_t)bh * L + row] = make_float2(m[c], z[c]);
    }
}

// -------------------------------------------------------------------------------------------------
// Forward, step 3, with the V rows in LDS: a work-group of sixteen wavefronts owns 1024 query rows of a head and walks
// the keys in ranges of 1024, whose V rows (128 KB) it loads once per range.  A group of eight lanes owns eight rows
// (their {maximum, 1 / denominator} and lane s's 16 bytes of their O rows in registers) and walks each row's remainder
// entries eight at a time: lane s fetches the s-th entry's raw logit, column and position and writes its probability
// (through the cache: a row's probabilities leave in pieces of at most eight as the ranges go by), the eight
// {column, probability} go round the group as in the column pass above.
// -------------------------------------------------------------------------------------------------
constexpr int HYB_RL_ROWS = 1024, HYB_RL_KEYS = 1024, HYB_RL_THREADS = 1024;
template <bool ST>
__global__ __launch_bounds__(HYB_RL_THREADS) void hyb_rem_pv_lds_kernel(
    const float* __restrict__ V, const float* __restrict__ Raw, float* __restrict__ P, float* __restrict__ O,
    float* __restrict__ Ocache, const float2* __restrict__ Stats, HybIndex ix, int L, int NB, int nnz, Layouts ly) {
    __shared__ f32x4 sv[HYB_RL_KEYS * 8];
    const int nrg = L / HYB_RL_ROWS;
    const int item = xcd_remap((int)blockIdx.x, (int)gridDim.x);  // the work-groups of a head share an XCD's L2
    const int bh = item / nrg, rg = item % nrg;
    const int t = threadIdx.x, grp = t >> 3, sub = t & 7, lane = t & 63;
    size_t ib, ob;
    int ild, old_;
    hyb_head<ST>(ly.in, ly.H, bh, L, ib, ild);
    hyb_head<ST>(ly.out, ly.H, bh, L, ob, old_);
    float* Ph = P + (size_t)bh * nnz;
    const float* raw = Raw + (size_t)bh * ix.nr;
    constexpr int NR = HYB_RL_ROWS / (HYB_RL_THREADS / 8);  // rows per lane group: 8
    f32x4 acc[NR];
    float2 st[NR];
    int e[NR], eend[NR];
#pragma unroll
    for (int c = 0; c < NR; ++c) {
        const int row = rg * HYB_RL_ROWS + c * (HYB_RL_THREADS / 8) + grp;
        acc[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
        st[c] = Stats[(size_t)bh * L + row];
        e[c] = ix.r_off[row];
        eend[c] = ix.r_off[row + 1];
    }
    for (int k0 = 0; k0 < L; k0 += HYB_RL_KEYS) {
        __syncthreads();  // everybody has finished with the previous range
#pragma unroll
        for (int k = 0; k < HYB_RL_KEYS * 8 / HYB_RL_THREADS; ++k) {
            const int idx = t + k * HYB_RL_THREADS;
            sv[idx] = reinterpret_cast<const f32x4*>(V + ib + (size_t)(k0 + (idx >> 3)) * ild)[idx & 7];
        }
        __syncthreads();
        const int kend = k0 + HYB_RL_KEYS;
#pragma unroll
        for (int c = 0; c < NR; ++c) {
            int nn = 8;
            while (nn == 8) {
                const int my = e[c] + sub;
                const int col = my < eend[c] ? ix.r_col[my] : 0x7fffffff;
                const bool in = col < kend;
                // columns ascend along the list: the entries of this range among the eight are the first nn
                nn = __popcll((__ballot(in) >> (lane & 56)) & 0xffull);
                if (nn == 0) break;
                float wgt = 0.f;
                int lcol = 0;
                if (in) {
                    wgt = __builtin_amdgcn_exp2f(raw[my] - st[c].x) * st[c].y;
                    Ph[ix.r_pos[my]] = wgt;
                    lcol = col - k0;
                }
                const int wx = __float_as_int(wgt);
                const int mcol = hyb_dpp<0x141>(lcol), mx = hyb_dpp<0x141>(wx);
#define SPION_HYB_ENTRY(CTRL, C, X) acc[c] += sv[hyb_dpp<CTRL>(C) * 8 + sub] * __int_as_float(hyb_dpp<CTRL>(X));
                SPION_HYB_ENTRY(0x00, lcol, wx)
                SPION_HYB_ENTRY(0x55, lcol, wx)
                SPION_HYB_ENTRY(0xaa, lcol, wx)
                SPION_HYB_ENTRY(0xff, lcol, wx)
                SPION_HYB_ENTRY(0x00, mcol, mx)
                SPION_HYB_ENTRY(0x55, mcol, mx)
                SPION_HYB_ENTRY(0xaa, mcol, mx)
                SPION_HYB_ENTRY(0xff, mcol, mx)
#undef SPION_HYB_ENTRY
                e[c] += nn;
            }
        }
    }
#pragma unroll
    for (int c = 0; c < NR; ++c) {
        const int row = rg * HYB_RL_ROWS + c * (HYB_RL_THREADS / 8) + grp;
        if (eend[c] == ix.r_off[row]) continue;  // a row without remainder entries
        f32x4* orow = reinterpret_cast<f32x4*>(O + ob + (size_t)row * old_) + sub;
        const f32x4 sum = *orow + acc[c];
        *orow = sum;
        if (Ocache) reinterpret_cast<f32x4*>(Ocache + ((size_t)bh * L + row) * 32)[sub] = sum;  // own copy: contiguous
    }
}

}  // namespace spion
