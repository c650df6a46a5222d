// Sparse attention (forward + backward) on an element-level CSR pattern for gfx950 (MI355X).
//
// Two kernel families serve the same C ABI:
//   * tile path    -- the pattern is a union of aligned 32x32 tiles (what a block mask of block size
//                     32, 64, ... expands to).  Every contraction is a dense 32x32xd product done with
//                     v_mfma_f32_32x32x2_f32; operands go straight from global memory into the MFMA
//                     register layout (every access is a coalesced 128-byte row segment), the tile
//                     list of a block row / block column is walked per wavefront.
//   * element path -- any other CSR (element-sparse patterns, odd head sizes): one wavefront per
//                     row gathers K/V rows; a transposed (CSC) index built on the host once per
//                     pattern makes dK/dV deterministic without atomics.
//
// Semantics follow the reference kernels (models/block_attn.cu:33-130, models/block_attn_mask.cu:88-173):
// the softmax denominator counts every off-pattern key with logit 0.
#include "common.h"
#include "tile_kernels.h"
#include "bf16_kernels.h"
#include "hybrid_kernels.h"
#include "../../include/spion_hip.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <queue>
#include <vector>

namespace spion {

// =================================================================================================
// element path
// =================================================================================================
constexpr int ELEM_WAVES = 4;

// [NB][D][L] -> [NB][L][D]
__global__ __launch_bounds__(256) void transpose_dl_kernel(const float* __restrict__ Xt, float* __restrict__ X,
                                                           int D, int L) {
    __shared__ float tile[32][33];
    const size_t base = (size_t)blockIdx.z * D * L;
    const int l0 = blockIdx.x * 32, d0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8) {
        int dd = d0 + r, ll = l0 + tx;
        tile[r][tx] = (dd < D && ll < L) ? Xt[base + (size_t)dd * L + ll] : 0.f;
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        int ll = l0 + r, dd = d0 + tx;
        if (ll < L && dd < D) X[base + (size_t)ll * D + dd] = tile[tx][r];
    }
}

template <int D>
__device__ __forceinline__ float row_dot(const float* __restrict__ a, const float* __restrict__ b) {
    float s = 0.f;
    const float4* a4 = reinterpret_cast<const float4*>(a);
    const float4* b4 = reinterpret_cast<const float4*>(b);
#pragma unroll
    for (int t = 0; t < D / 4; ++t) {
        float4 x = a4[t], y = b4[t];
        s = fmaf(x.x, y.x, s);
        s = fmaf(x.y, y.y, s);
        s = fmaf(x.z, y.z, s);
        s = fmaf(x.w, y.w, s);
    }
    return s;
}

// (Head size 128 only; smaller heads use the LDS-free primitives of gather_ops.h.)
// acc += sum_k w_k * X[col_k][:] over the entries of one CSR row, the entries being held one per lane in chunks
// of 64 (w_l, col_l).  VEC floats per lane: D/VEC lanes cover one X row and 64*VEC/D entries are processed per load
// instruction.  16-byte loads (eight entries per instruction at d = 32) because the vector-memory path charges per
// instruction and per row touched, not per byte: with four-byte loads, 32 lanes to a row, configuration 4 took
// 3.98 ms instead of 3.21 ms.
template <int D, int VEC = 4>
struct RowAcc {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    static constexpr int LPR = D / VEC;
    static constexpr int G = 64 / LPR;
    vec_t acc;
    __device__ __forceinline__ void clear() { acc = (vec_t)(0.f); }
    __device__ __forceinline__ void chunk(float w_l, int row_l, int nk, const float* __restrict__ X, int ld,
                                          int lane) {
        const int grp = lane / LPR, cl = lane % LPR;
        // Uniform trip count: every lane takes part in every shuffle.  Slots past nk carry w = 0
        // and row 0 (set by the caller), so they add nothing.
        constexpr int UN = G >= 8 ? 4 : 8;  // gathers in flight per lane before the first one is consumed
        for (int kb = 0; kb < nk; kb += UN * G) {
            float w[UN];
            const vec_t* xr[UN];
#pragma unroll
            for (int j = 0; j < UN; ++j) {
                const int kk = kb + j * G + grp;  // < 64 + UN*G: shuffles wrap, slots past nk are zero weights
                w[j] = __shfl(w_l, kk & 63, 64);
                const int rr = __shfl(row_l, kk & 63, 64);
                if (kb + j * G >= 64) w[j] = 0.f;
                xr[j] = reinterpret_cast<const vec_t*>(X + (size_t)rr * ld) + cl;
            }
            vec_t x[UN];
#pragma unroll
            for (int j = 0; j < UN; ++j) x[j] = *xr[j];
#pragma unroll
            for (int j = 0; j < UN; ++j)
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] = fmaf(w[j], x[j][e], acc[e]);
        }
    }
    __device__ __forceinline__ void finish(float* __restrict__ out_row, int lane) {
        vec_t a = acc;
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1)
#pragma unroll
            for (int e = 0; e < VEC; ++e) a[e] += __shfl_xor(a[e], o, 64);
        if (lane < LPR) reinterpret_cast<vec_t*>(out_row)[lane] = a;
    }
};

// One wavefront per (head, row).  K is row-major here ([NB][L][D], transposed copy in the workspace).  ST: the heads
// are [B][H][L][D] views located by `ly` (head_slice) instead of contiguous slices.
template <int D, bool MASK, bool ST>
__global__ __launch_bounds__(64 * ELEM_WAVES) __attribute__((amdgpu_waves_per_eu(D <= 32 ? 6 : D == 64 ? 3 : 2, 8))) void elem_fwd_kernel(
    const float* __restrict__ Q, const float* __restrict__ K, const float* __restrict__ V,
    const float* __restrict__ pen, float* __restrict__ P, float* __restrict__ O,
    const int* __restrict__ offs, const int* __restrict__ cols, int L, int NB, int nnz, float scale, Layouts ly) {
    const int lane = threadIdx.x & 63;
    // consecutive rows (which gather overlapping K/V rows and share lines of P) on the same XCD
    const long long wrow = (long long)xcd_remap((int)blockIdx.x, (int)gridDim.x) * ELEM_WAVES + (threadIdx.x >> 6);
    if (wrow >= (long long)NB * L) return;
    const int bh = (int)(wrow / L), row = (int)(wrow % L);
    const int r0 = offs[row], cnt = offs[row + 1] - r0;
    size_t ib, ob, bytes;
    int ild, old_;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, bytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, bytes);
    const float* q = Q + ib + (size_t)row * ild;
    float* p = P + (size_t)bh * nnz + r0;
    const int* cj = cols + r0;

    float m = MASK ? 0.f : -100.f;
    if constexpr (D <= 64) {
        // LDS-free gathers (gather_ops.h): the chunk's entries follow the lane order of the gather groups
        constexpr int LPR = D / 4, KEEP = 2;
        const int ent = gather_entry_of_lane<LPR>(lane);
        const f32x4 q4 = reinterpret_cast<const f32x4*>(q)[lane % LPR];
        float vk[KEEP];  // the logits of the first chunks stay in registers; longer rows go back to what they stored
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int k = c0 + ent;
            const int col = k < cnt ? cj[k] : 0;
            float v = gather_dot<LPR>(q4, K + ib, ild, col, min(64, cnt - c0), lane) * scale;
            if (k < cnt) {
                if (MASK) v -= pen[(size_t)bh * L + col];
                p[k] = v;
                m = fmaxf(m, v);
            }
#pragma unroll
            for (int c = 0; c < KEEP; ++c)
                if (c0 == 64 * c) vk[c] = v;
        }
        m = wave_max(m);
        float z = 0.f;
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int k = c0 + ent;
            float v = 0.f;
#pragma unroll
            for (int c = 0; c < KEEP; ++c)
                if (c0 == 64 * c) v = vk[c];
            if (c0 >= 64 * KEEP && k < cnt) v = p[k];
            if (k < cnt) z += __expf(v - m);
        }
        z = wave_sum(z);
        z += (float)(L - cnt) * __expf(-m);
        const float r = 1.0f / z;
        GatherRowAcc<LPR> acc;
        acc.clear();
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int k = c0 + ent;
            float v = 0.f, w = 0.f;
#pragma unroll
            for (int c = 0; c < KEEP; ++c)
                if (c0 == 64 * c) v = vk[c];
            int col = 0;
            if (k < cnt) {
                if (c0 >= 64 * KEEP) v = p[k];
                w = __expf(v - m) * r;
                col = cj[k];
                p[k] = w;
            }
            acc.chunk(w, col, min(64, cnt - c0), V + ib, ild, lane);
        }
        const f32x4 tot = acc.total();
        if (lane < LPR) reinterpret_cast<f32x4*>(O + ob + (size_t)row * old_)[lane] = tot;
    } else {
        for (int k = lane; k < cnt; k += 64) {
            int col = cj[k];
            float v = row_dot<D>(q, K + ib + (size_t)col * ild) * scale;
            if (MASK) v -= pen[(size_t)bh * L + col];
            p[k] = v;
            m = fmaxf(m, v);
        }
        m = wave_max(m);
        float z = 0.f;
        for (int k = lane; k < cnt; k += 64) z += __expf(p[k] - m);
        z = wave_sum(z);
        z += (float)(L - cnt) * __expf(-m);
        const float r = 1.0f / z;

        RowAcc<D> acc;
        acc.clear();
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int k = c0 + lane;
            float w = 0.f;
            int col = 0;
            if (k < cnt) {
                w = __expf(p[k] - m) * r;
                col = cj[k];
                p[k] = w;
            }
            acc.chunk(w, col, min(64, cnt - c0), V + ib, ild, lane);
        }
        acc.finish(O + ob + (size_t)row * old_, lane);
    }
}

// Row pass of the backward: dP = dO.V^T on the pattern, g = sum_row dP*P, dS = (dP*P - P*g)*scale
// (written to the caller's dS scratch for the column pass), dQ = dS.K.
template <int D, bool ST>
__global__ __launch_bounds__(64 * ELEM_WAVES) __attribute__((amdgpu_waves_per_eu(D <= 32 ? 6 : D == 64 ? 3 : 2, 8))) void elem_bwd_row_kernel(
    const float* __restrict__ K, const float* __restrict__ V, const float* __restrict__ P,
    const float* __restrict__ dO, float* __restrict__ dS, float* __restrict__ dQ,
    const int* __restrict__ offs, const int* __restrict__ cols, int L, int NB, int nnz, float scale, Layouts ly) {
    const int lane = threadIdx.x & 63;
    // consecutive rows (which gather overlapping K/V rows and share lines of P) on the same XCD
    const long long wrow = (long long)xcd_remap((int)blockIdx.x, (int)gridDim.x) * ELEM_WAVES + (threadIdx.x >> 6);
    if (wrow >= (long long)NB * L) return;
    const int bh = (int)(wrow / L), row = (int)(wrow % L);
    const int r0 = offs[row], cnt = offs[row + 1] - r0;
    size_t ib, ob, gb, bytes;
    int ild, old_, gld;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, bytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, bytes);
    head_slice<ST, D>(ly.grad, ly.H, bh, L, gb, gld, bytes);
    const float* go = dO + ob + (size_t)row * old_;
    const float* p = P + (size_t)bh * nnz + r0;
    float* ds = dS + (size_t)bh * nnz + r0;
    const int* cj = cols + r0;

    float g = 0.f;
    if constexpr (D <= 64) {
        constexpr int LPR = D / 4, KEEP = 2;
        const int ent = gather_entry_of_lane<LPR>(lane);
        const f32x4 go4 = reinterpret_cast<const f32x4*>(go)[lane % LPR];
        float tk[KEEP], pk[KEEP];  // dP*P and P of the first chunks stay in registers
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int k = c0 + ent;
            const int col = k < cnt ? cj[k] : 0;
            const float dp = gather_dot<LPR>(go4, V + ib, ild, col, min(64, cnt - c0), lane);
            float t = 0.f, pv = 0.f;
            if (k < cnt) {
                pv = p[k];
                t = dp * pv;
                if (c0 >= 64 * KEEP) ds[k] = t;
                g += t;
            }
#pragma unroll
            for (int c = 0; c < KEEP; ++c)
                if (c0 == 64 * c) {
                    tk[c] = t;
                    pk[c] = pv;
                }
        }
        g = wave_sum(g);
        GatherRowAcc<LPR> acc;
        acc.clear();
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int k = c0 + ent;
            float t = 0.f, pv = 0.f, w = 0.f;
#pragma unroll
            for (int c = 0; c < KEEP; ++c)
                if (c0 == 64 * c) {
                    t = tk[c];
                    pv = pk[c];
                }
            int col = 0;
            if (k < cnt) {
                if (c0 >= 64 * KEEP) {
                    t = ds[k];
                    pv = p[k];
                }
                w = (t - pv * g) * scale;
                col = cj[k];
                ds[k] = w;
            }
            acc.chunk(w, col, min(64, cnt - c0), K + ib, ild, lane);
        }
        const f32x4 tot = acc.total();
        if (lane < LPR) reinterpret_cast<f32x4*>(dQ + gb + (size_t)row * gld)[lane] = tot;
    } else {
        for (int k = lane; k < cnt; k += 64) {
            float t = row_dot<D>(go, V + ib + (size_t)cj[k] * ild) * p[k];
            ds[k] = t;
            g += t;
        }
        g = wave_sum(g);

        RowAcc<D> acc;
        acc.clear();
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int k = c0 + lane;
            float w = 0.f;
            int col = 0;
            if (k < cnt) {
                w = (ds[k] - p[k] * g) * scale;
                col = cj[k];
                ds[k] = w;
            }
            acc.chunk(w, col, min(64, cnt - c0), K + ib, ild, lane);
        }
        acc.finish(dQ + gb + (size_t)row * gld, lane);
    }
}

// Column pass of the backward: dK_j = sum_i dS_ij Q_i, dV_j = sum_i P_ij dO_i over the transposed index.
template <int D, bool ST>
__global__ __launch_bounds__(64 * ELEM_WAVES) void elem_bwd_col_kernel(
    const float* __restrict__ Q, const float* __restrict__ dO, const float* __restrict__ P,
    const float* __restrict__ dS, float* __restrict__ dK, float* __restrict__ dV,
    const int* __restrict__ colptr, const int* __restrict__ crow, const int* __restrict__ cpos, int L, int NB,
    int nnz, Layouts ly) {
    const int lane = threadIdx.x & 63;
    // consecutive columns on the same XCD: the 32 columns whose entries in a row share a 128-byte line of P and
    // dS then share it in one L2 instead of fetching it into eight
    const long long wcol = (long long)xcd_remap((int)blockIdx.x, (int)gridDim.x) * ELEM_WAVES + (threadIdx.x >> 6);
    if (wcol >= (long long)NB * L) return;
    const int bh = (int)(wcol / L), col = (int)(wcol % L);
    const int c0p = colptr[col], cnt = colptr[col + 1] - c0p;
    size_t ib, ob, gb, bytes;
    int ild, old_, gld;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, bytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, bytes);
    head_slice<ST, D>(ly.grad, ly.H, bh, L, gb, gld, bytes);
    const float* p = P + (size_t)bh * nnz;
    const float* ds = dS + (size_t)bh * nnz;

    if constexpr (D <= 64) {
        constexpr int LPR = D / 4;
        const int ent = gather_entry_of_lane<LPR>(lane);
        GatherRowAcc<LPR> ak, av;
        ak.clear();
        av.clear();
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int e = c0 + ent;
            float wk = 0.f, wv = 0.f;
            int row = 0;
            if (e < cnt) {
                int pos = cpos[c0p + e];
                row = crow[c0p + e];
                wk = ds[pos];
                wv = p[pos];
            }
            const int nk = min(64, cnt - c0);
            ak.chunk(wk, row, nk, Q + ib, ild, lane);
            av.chunk(wv, row, nk, dO + ob, old_, lane);
        }
        const f32x4 tk = ak.total(), tv = av.total();
        if (lane < LPR) {
            reinterpret_cast<f32x4*>(dK + gb + (size_t)col * gld)[lane] = tk;
            reinterpret_cast<f32x4*>(dV + gb + (size_t)col * gld)[lane] = tv;
        }
    } else {
        RowAcc<D> ak, av;
        ak.clear();
        av.clear();
        for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int e = c0 + lane;
            float wk = 0.f, wv = 0.f;
            int row = 0;
            if (e < cnt) {
                int pos = cpos[c0p + e];
                row = crow[c0p + e];
                wk = ds[pos];
                wv = p[pos];
            }
            const int nk = min(64, cnt - c0);
            ak.chunk(wk, row, nk, Q + ib, ild, lane);
            av.chunk(wv, row, nk, dO + ob, old_, lane);
        }
        ak.finish(dK + gb + (size_t)col * gld, lane);
        av.finish(dV + gb + (size_t)col * gld, lane);
    }
}

// =================================================================================================
// host side
// =================================================================================================
// Device side of a schedule of the bf16 kernels (build_bf16_plan): the lists, the number of persistent wavefronts,
// the workspace slots of the chunks of long strips and {strip, first slot, chunks, tiles} per long strip.
struct Bf16Plan {
    Bf16Sched sched{};
    const int* d_longs = nullptr;
    int lanes = 0, slots = 0, n_long = 0;
};

struct PatternIndex {
    const int* key_off = nullptr;
    const int* key_col = nullptr;
    int key_nnz = -1;
    bool valid = false;
    bool tiled = false;
    int ntiles = 0;
    int max_row_tiles = 0, max_col_tiles = 0;
    int n_fwd_long = 0;  // strips of more than 16 tiles: the first entries of the forward's strip order
    int n_fwd_long24 = 0;  // strips of more than 24 tiles
    // block rows / block columns longer than long_strip_threshold (global rows and columns): the first entries of
    // the row pass's and of the column pass's strip order
    int n_long_rows = 0, n_long_cols = 0;
    int* d_blob = nullptr;  // one allocation holding every array below
    int *d_trp = nullptr, *d_tcol = nullptr, *d_tcp = nullptr;
    int* d_tcdesc = nullptr;  // per tile of the transposed index: {block row I, offset of the tile in P, row stride, 0}
    // per strip in launch order, {strip, first tile, tiles, P offset}: row pass, forward, column pass
    int *d_rdesc = nullptr, *d_fdesc = nullptr, *d_cdesc = nullptr;
    // bf16 family: schedules of persistent wavefronts over block rows, pairs of block rows and block columns
    Bf16Plan plan_row, plan_pair, plan_col;
    int *d_ccp = nullptr, *d_crow = nullptr, *d_cpos = nullptr;
    // element-sparse pattern whose well-filled 32x32 tiles run on the MFMA units (hybrid_kernels.h)
    bool hybrid = false;
    int hyb_tiles = 0, hyb_nr = 0;
    HybIndex hyb{};
    void release() {
        if (d_blob) (void)hipFree(d_blob);
        *this = PatternIndex();
    }
};

struct SparseAttn {
    HandleHeader hdr;
    int d, L, NB, bs;
    bool has_mask;
    float scale;
    // Analysed patterns, keyed by (Offsets pointer, Columns pointer, nnz): a handle that alternates between a few
    // masks (one per layer, or train / eval masks) analyses each once.  `pat` is a non-owning view of the slot in
    // use; the slots own the device memory.  A key says nothing about the arrays' contents: whoever frees or
    // rewrites index arrays must drop the key (spion_forget_pattern / spion_invalidate_pattern).
    static constexpr int PAT_SLOTS = 8;
    PatternIndex pats[PAT_SLOTS];
    uint64_t pat_stamp[PAT_SLOTS] = {};
    uint64_t pat_clock = 0;
    int analyses_from_device = 0, analyses_from_host = 0;  // counted for tests
    PatternIndex pat;
    void release_patterns() {
        for (auto& p : pats) p.release();
        pat = PatternIndex();
    }
    float* ws_rowsum = nullptr;  // [NB][L]   g of the backward (tile path)
    // Copies of O kept by the forward of the tile path, keyed by the Attn (P) buffer that forward
    // filled: a backward that is handed the same P pointer gets its row sums g_i = dO_i . O_i from the
    // copy in one cheap step instead of a sweep over all tiles.  The key is sound because a forward that
    // overwrites a P buffer also overwrites the copy filed under it; an unknown P pointer simply takes the
    // two-sweep kernel.
    static constexpr int O_SLOTS = 4;
    struct OSlot {
        const float* key = nullptr;
        float* buf = nullptr;
        uint64_t stamp = 0;
    } oslot[O_SLOTS];
    uint64_t ostamp = 0;
    bool use_ocache = true;
    float* ws_trans = nullptr;   // [NB][L][d] row-major copy of the transposed operand (element path)
    float* ws_stats = nullptr;   // [NB][L][2] softmax row statistics handed between the hybrid forward's launches
    float* ws_raw = nullptr;     // [NB][nr] raw logits of a hybrid pattern's remainder, forward only
    size_t ws_raw_count = 0;
    float* ws_ds = nullptr;      // [NB][nnz] dS scratch of the strided backward on patterns without tile structure
    size_t ws_ds_count = 0;
    float* ws_part = nullptr;    // [NB][slots][slot floats] partial results of the chunks of long strips (bf16 family)
    size_t ws_part_floats = 0;
    // Side stream (default priority) of the fp32 tile passes on a pattern with a few long strips: the long strips'
    // launch goes to the caller's stream, the launch of all other strips to this one, beside it; forked from and
    // joined to the caller's stream by the two events.  Created when such a pattern is analysed, never inside a call.
    hipStream_t side = nullptr;
    hipEvent_t side_fork = nullptr, side_join = nullptr;
    bool ensure_side() {
        if (side) return true;
        if (hipStreamCreateWithFlags(&side, hipStreamNonBlocking) != hipSuccess) return side = nullptr, false;
        if (hipEventCreateWithFlags(&side_fork, hipEventDisableTiming) != hipSuccess ||
            hipEventCreateWithFlags(&side_join, hipEventDisableTiming) != hipSuccess) {
            (void)hipStreamDestroy(side);
            return side = nullptr, false;
        }
        return true;
    }
    // Buffers a grown workspace has replaced.  They stay allocated until the handle is destroyed: a HIP graph
    // recorded earlier on this handle has their addresses in its kernel nodes and may still be replayed.
    std::vector<void*> retired;
    int last_path = 0;
    bool is_bf16 = false;  // handle of the bf16 family: tile patterns only, P is never materialised
    bool force_element = false;
    int bwd_passes = 3;  // bit 0: row pass (g, dQ), bit 1: column pass (dK, dV); profiling only
};

static SparseAttn* as_sparse(void* h, const char* who) {
    SparseAttn* a = static_cast<SparseAttn*>(h);
    note_current_handle(a && a->hdr.magic == KIND_SPARSE ? &a->hdr : nullptr);
    if (!a || a->hdr.magic != KIND_SPARSE) {
        set_error("%s: not a sparse-attention handle", who);
        return nullptr;
    }
    return a;
}

static bool tile_supported(int d) { return d == 32 || d == 64; }
static bool elem_supported(int d) { return d == 16 || d == 32 || d == 64 || d == 128; }

static float* noalloc_scratch(bool report);

void* sparse_init(int emb_dim, int seq_len, int num_batches, int block_size, bool has_mask) {
    if (emb_dim <= 0 || seq_len <= 0 || num_batches <= 0) {
        set_error("init: emb_dim, seq_len and num_batches must be positive (got %d, %d, %d)", emb_dim, seq_len,
                  num_batches);
        return nullptr;
    }
    if (!elem_supported(emb_dim)) {
        set_error("init: emb_dim %d unsupported (16, 32, 64 or 128)", emb_dim);
        return nullptr;
    }
    if ((long long)emb_dim * seq_len >= (1LL << 29)) {  // 32-bit byte offsets into one head's [L][d] slice
        set_error("init: seq_len %d x emb_dim %d too large (one head's slice must stay under 2 GiB)", seq_len, emb_dim);
        return nullptr;
    }
    SparseAttn* a = new SparseAttn();
    a->hdr.magic = KIND_SPARSE;
    a->hdr.stream = nullptr;
    a->hdr.err[0] = 0;
    a->d = emb_dim;
    a->L = seq_len;
    a->NB = num_batches;
    a->bs = block_size;
    a->has_mask = has_mask;
    a->scale = 1.0f / sqrtf((float)emb_dim);  // models/block_attn.cu:420
    (void)noalloc_scratch(false);  // per-device address of the built-in scratch array, looked up once
    return a;
}

void sparse_destroy(void* h) {
    SparseAttn* a = as_sparse(h, "destroy");
    if (!a) return;
    a->release_patterns();
    if (a->side) {
        (void)hipStreamSynchronize(a->side);
        (void)hipEventDestroy(a->side_fork);
        (void)hipEventDestroy(a->side_join);
        (void)hipStreamDestroy(a->side);
    }
    if (a->ws_rowsum) (void)hipFree(a->ws_rowsum);
    if (a->ws_trans) (void)hipFree(a->ws_trans);
    if (a->ws_stats) (void)hipFree(a->ws_stats);
    if (a->ws_ds) (void)hipFree(a->ws_ds);
    if (a->ws_raw) (void)hipFree(a->ws_raw);
    if (a->ws_part) (void)hipFree(a->ws_part);
    for (void* p : a->retired) (void)hipFree(p);
    for (auto& sl : a->oslot)
        if (sl.buf) (void)hipFree(sl.buf);
    a->hdr.magic = 0;
    note_current_handle(nullptr);
    delete a;
}

// A strip counts as long (a global row or column) when it has more tiles than this.
static int long_strip_threshold(int nstrips, int ntiles) {
    const int avg = nstrips ? (ntiles + nstrips - 1) / nstrips : 0;
    return std::max(4 * avg + 8, 32);
}

// Schedule of the bf16 kernels.  A launch is a fixed set of persistent one-wavefront work-groups ("lanes of work");
// each walks a list of items built here, so that no lane outlasts the others by much and a lane's tile loads run
// on from one item into the next:
//   items    {strip, first tile (index into the tile list), tiles, kind} -- kind >= 0: a chunk of a long strip (a global
//            row or column, cut so that no item is much longer than the average lane's share) that leaves its partial
//            result in workspace slot `kind`; -1: a whole strip; -2: strips `strip` and `strip + 1`, which hold the
//            same tiles, walked together (forward only);
//   lane_ptr / lane_ent  CSR-like: lane s works on entries lane_ptr[s] .. lane_ptr[s+1]-1, each {head, item};
//   longs    {strip, first slot, chunks, tiles} per long strip, for the merge kernels.
// Lanes are dealt to the dies in turn (lane s runs on die s % 8, as work-groups are), and a die's lanes share the
// heads of that die one head after the other (the K/V of a head then stay in the die's L2); within a head the items
// go longest first to the lane with the least work so far.
struct Bf16PlanHost {
    std::vector<int> items, lane_ptr, lane_ent, longs;
    int slots = 0, lanes = 0;
};
static Bf16PlanHost build_bf16_plan(const std::vector<int>& ptr, int nstrips, bool pairs, int NB, int lanes_wanted) {
    Bf16PlanHost out;
    long long ntiles = 0;
    for (int i = 0; i < nstrips; ++i) ntiles += ptr[i + 1] - ptr[i];
    const int groups = NB % 8 == 0 ? 8 : 1;  // dies
    const int lanes = std::max(groups, lanes_wanted / groups * groups);
    // no item much longer than a lane's share of the launch, nor shorter than a few tiles
    const long long share = (ntiles * NB + lanes - 1) / lanes;
    const int avg = nstrips ? (int)((ntiles + nstrips - 1) / nstrips) : 0;
    const int long_len = (int)std::max<long long>(std::min<long long>(std::max(4 * avg + 8, 32), std::max<long long>(share / 2, 8)), 8);
    struct It {
        int strip, t0, n, kind;
    };
    std::vector<It> its;
    const int step = pairs ? 2 : 1;
    for (int i = 0; i < nstrips; i += step) {
        const int cnt = ptr[i + 1] - ptr[i];
        if (cnt <= long_len) {
            its.push_back({i, ptr[i], cnt, pairs ? -2 : -1});
            continue;
        }
        for (int k = 0; k < step; ++k) {  // long strips are cut one by one, also where strips are paired
            const int I = i + k, chunks = (cnt + long_len - 1) / long_len;
            out.longs.insert(out.longs.end(), {I, out.slots, chunks, cnt});
            for (int c = 0; c < chunks; ++c) {
                const int b = (int)((long long)cnt * c / chunks), e = (int)((long long)cnt * (c + 1) / chunks);
                its.push_back({I, ptr[I] + b, e - b, out.slots + c});
            }
            out.slots += chunks;
        }
    }
    std::vector<int> order(its.size());
    for (size_t i = 0; i < its.size(); ++i) order[i] = (int)i;
    const int unit = pairs ? 2 : 1;  // a pair does two strips' arithmetic per tile
    auto weight = [&](const It& x) { return (x.kind == -2 ? unit : 1) * x.n + 2; };
    std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return weight(its[x]) > weight(its[y]); });
    for (const It& x : its) out.items.insert(out.items.end(), {x.strip, x.t0, x.n, x.kind});
    if (out.items.empty()) out.items.assign(4, 0);
    // deal: per die, head after head, every item to the lane of that die with the least work so far
    const int per_group = lanes / groups, heads_per_group = NB / groups;
    std::vector<std::vector<int>> lane_list(lanes);
    for (int g = 0; g < groups; ++g) {
        typedef std::pair<long long, int> Load;  // (work so far, lane of this die)
        std::priority_queue<Load, std::vector<Load>, std::greater<Load>> heap;
        for (int j = 0; j < per_group; ++j) heap.push({0, j});
        for (int hh = 0; hh < heads_per_group; ++hh) {
            const int bh = g * heads_per_group + hh;
            for (int o : order) {
                Load top = heap.top();
                heap.pop();
                const int lane = top.second * groups + g;
                lane_list[lane].push_back(bh);
                lane_list[lane].push_back(o);
                top.first += weight(its[o]);
                heap.push(top);
            }
        }
    }
    out.lane_ptr.assign(1, 0);
    for (int sidx = 0; sidx < lanes; ++sidx) {
        out.lane_ent.insert(out.lane_ent.end(), lane_list[sidx].begin(), lane_list[sidx].end());
        out.lane_ptr.push_back((int)out.lane_ent.size() / 2);
    }
    if (out.lane_ent.empty()) out.lane_ent.assign(2, 0);
    out.lanes = lanes;
    return out;
}

// Wavefronts a launch of the bf16 kernels keeps resident: two per SIMD on every compute unit of the device.
// SPION_BF16_LANES (tests; read whenever a pattern is indexed) overrides the number: with a handful of lanes every
// lane walks many items of several heads even on a small problem.
static int bf16_lanes() {
    static int device_lanes = 0;
    if (!device_lanes) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            cus <= 0) {
            (void)hipGetLastError();
            cus = 256;
        }
        device_lanes = cus * 8;
    }
    if (const char* env = getenv("SPION_BF16_LANES")) return std::min(std::max(1, atoi(env)), 1 << 16);
    return device_lanes;
}

// Copy the index to the host once (unless the caller hands over host copies), validate it, detect the tile
// structure and build the transposed index.  Returns false (error recorded) if the CSR is inconsistent.
static bool analyse_pattern(SparseAttn* a, const int* Offsets, const int* Columns, int nnz,
                            const int* host_off = nullptr, const int* host_col = nullptr) {
    PatternIndex pi;
    const int L = a->L;
    if (nnz < 0) {
        set_error("pattern: nnz %d is negative", nnz);
        return false;
    }
    if (nnz >= (1 << 29)) {  // the kernels address one head's map with 32-bit byte offsets
        set_error("pattern: nnz %d too large (one head's map must stay under 2 GiB)", nnz);
        return false;
    }
    std::vector<int> off_copy, col_copy;
    if (!host_off || (nnz && !host_col)) {
        off_copy.resize(L + 1);
        col_copy.resize((size_t)nnz);
        if (!SPION_HIP_OK(hipMemcpyAsync(off_copy.data(), Offsets, sizeof(int) * (L + 1), hipMemcpyDeviceToHost,
                                         a->hdr.stream)))
            return false;
        if (nnz && !SPION_HIP_OK(hipMemcpyAsync(col_copy.data(), Columns, sizeof(int) * (size_t)nnz,
                                                hipMemcpyDeviceToHost, a->hdr.stream)))
            return false;
        if (!SPION_HIP_OK(hipStreamSynchronize(a->hdr.stream))) return false;
        host_off = off_copy.data();
        host_col = col_copy.data();
        a->analyses_from_device++;
    } else {
        a->analyses_from_host++;
    }
    const int* off = host_off;
    const int* col = host_col;

    if (off[0] != 0 || off[L] != nnz) {
        set_error("pattern: Offsets[0]=%d, Offsets[L]=%d do not match nnz=%d", off[0], off[L], nnz);
        return false;
    }
    for (int i = 0; i < L; ++i) {
        if (off[i + 1] < off[i]) {
            set_error("pattern: Offsets not monotone at row %d", i);
            return false;
        }
        for (int k = off[i]; k < off[i + 1]; ++k) {
            if (col[k] < 0 || col[k] >= L) {
                set_error("pattern: column %d out of range at row %d", col[k], i);
                return false;
            }
            if (k > off[i] && col[k] <= col[k - 1]) {
                set_error("pattern: columns of row %d are not strictly increasing", i);
                return false;
            }
        }
    }

    // --- tile detection: every 32-row strip has identical rows made of aligned runs of 32 columns
    bool tiled = !a->force_element && tile_supported(a->d) && (L % 32 == 0);
    const int nbr = L / 32;
    std::vector<int> trp, tcol;
    if (tiled) {
        trp.assign(nbr + 1, 0);
        for (int I = 0; I < nbr && tiled; ++I) {
            const int r0 = I * 32, a0 = off[r0], n0 = off[r0 + 1] - a0;
            if (n0 % 32) tiled = false;
            for (int k = 0; k < n0 && tiled; ++k) {
                int c = col[a0 + k];
                if ((k % 32 == 0 && c % 32 != 0) || (k % 32 && c != col[a0 + k - 1] + 1)) tiled = false;
            }
            for (int r = 1; r < 32 && tiled; ++r) {
                const int ar = off[r0 + r];
                if (off[r0 + r + 1] - ar != n0 || (n0 && memcmp(&col[ar], &col[a0], sizeof(int) * n0))) tiled = false;
            }
            if (tiled) {
                for (int k = 0; k < n0; k += 32) tcol.push_back(col[a0 + k] / 32);
                trp[I + 1] = (int)tcol.size();
            }
        }
    }

    std::vector<int> blob;
    auto append = [&](const std::vector<int>& v) {
        size_t o = blob.size();
        blob.insert(blob.end(), v.begin(), v.end());
        while (blob.size() % 4) blob.push_back(0);
        return o;
    };
    size_t o_trp = 0, o_tcol = 0, o_tcp = 0, o_tcdesc = 0, o_ccp = 0, o_crow = 0, o_cpos = 0;
    size_t o_rdesc = 0, o_fdesc = 0, o_cdesc = 0;
    size_t o_plan[3][4] = {};
    size_t hyb_off[14] = {};
    if (tiled) {
        const int nt = (int)tcol.size();
        std::vector<int> tcp(nbr + 1, 0), tcdesc(4 * (size_t)std::max(nt, 1), 0);
        for (int t = 0; t < nt; ++t) tcp[tcol[t] + 1]++;
        for (int J = 0; J < nbr; ++J) tcp[J + 1] += tcp[J];
        std::vector<int> fill(tcp.begin(), tcp.end() - 1);
        int mr = 0, mc = 0;
        for (int I = 0; I < nbr; ++I) {
            mr = std::max(mr, trp[I + 1] - trp[I]);
            for (int t = trp[I]; t < trp[I + 1]; ++t) {
                int e = fill[tcol[t]]++;
                tcdesc[4 * (size_t)e + 0] = I;
                tcdesc[4 * (size_t)e + 1] = off[I * 32] + (t - trp[I]) * 32;
                tcdesc[4 * (size_t)e + 2] = (trp[I + 1] - trp[I]) * 32;
            }
        }
        for (int J = 0; J < nbr; ++J) mc = std::max(mc, tcp[J + 1] - tcp[J]);
        Bf16PlanHost plan_r, plan_p, plan_c;
        if (a->is_bf16) {
            // strips 2k and 2k+1 with the same block columns (masks of 64 x 64 blocks and larger): the forward
            // gives one wavefront both strips of a pair
            bool pairs = nbr % 2 == 0 && nt > 0;
            for (int k = 0; pairs && k < nbr / 2; ++k) {
                const int a0 = trp[2 * k], a1 = trp[2 * k + 1], n0 = a1 - a0, n1 = trp[2 * k + 2] - a1;
                pairs = n0 == n1 && std::equal(tcol.begin() + a0, tcol.begin() + a1, tcol.begin() + a1);
            }
            plan_r = build_bf16_plan(trp, nbr, false, a->NB, bf16_lanes());
            plan_c = build_bf16_plan(tcp, nbr, false, a->NB, bf16_lanes());
            if (pairs) plan_p = build_bf16_plan(trp, nbr, true, a->NB, bf16_lanes());
        }
        // Behind each pointer array: the order the fp32 kernels walk the strips of a head in.  Strips are
        // bucketed by length class -- rows: more than 2 MAXT tiles of the forward's register budget, more than
        // MAXT, the rest; columns: long ones, the rest -- so that long strips start first,
        // and keep their index order inside a bucket (neighbouring strips share K/V tiles in the caches).
        const int maxt = a->d == 32 ? 8 : 4, long_len = long_strip_threshold(nbr, nt);
        auto append_order = [&](std::vector<int>& ptr, bool rows) {
            std::vector<int> order(nbr);
            for (int i = 0; i < nbr; ++i) order[i] = i;
            auto bucket = [&](int i) {
                const int len = ptr[i + 1] - ptr[i];
                if (rows) return len > long_len ? -1 : len > 2 * maxt ? 0 : len > maxt ? 1 : 2;
                return len > long_len ? 0 : 1;
            };
            for (int i = 0; i < nbr; ++i)
                if (ptr[i + 1] - ptr[i] > long_len) (rows ? pi.n_long_rows : pi.n_long_cols)++;
            std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return bucket(x) < bucket(y); });
            ptr.insert(ptr.end(), order.begin(), order.end());
        };
        append_order(trp, true);
        append_order(tcp, false);
        // One 16-byte descriptor per strip in launch order, {strip, first tile, tiles, offset of the strip's first
        // element in a head's P}: a work-group learns everything about its strip from one scalar load instead of
        // three dependent ones.  The row pass walks the bucketed order above.  The forward and the column pass
        // walk the strips by descending length (equal lengths in index order): the launch then ends on the
        // shortest strips.  Measured: on one machine the north star's column pass went 0.203 -> 0.193 ms and the
        // forward -1 %, on another neither moved; one round of 512 work-groups at L = 1024: forward 0.0094 ->
        // 0.0088 ms; the row pass is 0-3 % slower in that order on the large shapes, hence its own.
        auto by_length = [&](const std::vector<int>& ptr) {
            std::vector<int> order(nbr);
            for (int i = 0; i < nbr; ++i) order[i] = i;
            std::stable_sort(order.begin(), order.end(),
                             [&](int x, int y) { return ptr[x + 1] - ptr[x] > ptr[y + 1] - ptr[y]; });
            return order;
        };
        const std::vector<int> rows_sorted = by_length(trp), cols_sorted = by_length(tcp);
        std::vector<int> rdesc(4 * (size_t)nbr), fdesc(4 * (size_t)nbr), cdesc(4 * (size_t)nbr);
        for (int p = 0; p < nbr; ++p) {
            const int I = trp[nbr + 1 + p], F = rows_sorted[p], J = cols_sorted[p];
            rdesc[4 * p + 0] = I;
            rdesc[4 * p + 1] = trp[I];
            rdesc[4 * p + 2] = trp[I + 1] - trp[I];
            rdesc[4 * p + 3] = off[I * 32];
            fdesc[4 * p + 0] = F;
            fdesc[4 * p + 1] = trp[F];
            fdesc[4 * p + 2] = trp[F + 1] - trp[F];
            fdesc[4 * p + 3] = off[F * 32];
            cdesc[4 * p + 0] = J;
            cdesc[4 * p + 1] = tcp[J];
            cdesc[4 * p + 2] = tcp[J + 1] - tcp[J];
            cdesc[4 * p + 3] = 0;
        }
        if (pi.n_long_rows > 0 || pi.n_long_cols > 0) (void)a->ensure_side();  // see launch_tile_bwd
        for (int p = 0; p < nbr; ++p)
            if (fdesc[4 * p + 2] > 16) pi.n_fwd_long++;
        for (int p = 0; p < nbr; ++p)
            if (fdesc[4 * p + 2] > 24) pi.n_fwd_long24++;
        o_rdesc = append(rdesc);
        o_fdesc = append(fdesc);
        o_cdesc = append(cdesc);
        auto file_plan = [&](const Bf16PlanHost& ph, Bf16Plan& dst, size_t (&o)[4]) {
            dst.lanes = ph.lanes;
            dst.slots = ph.slots;
            dst.n_long = (int)ph.longs.size() / 4;
            if (!ph.lanes) return;
            o[0] = append(ph.items);
            o[1] = append(ph.lane_ptr);
            o[2] = append(ph.lane_ent);
            o[3] = append(ph.longs);
        };
        file_plan(plan_r, pi.plan_row, o_plan[0]);
        file_plan(plan_p, pi.plan_pair, o_plan[1]);
        file_plan(plan_c, pi.plan_col, o_plan[2]);
        if (tcol.empty()) tcol.push_back(0);
        o_trp = append(trp);
        o_tcol = append(tcol);
        o_tcp = append(tcp);
        o_tcdesc = append(tcdesc);
        pi.ntiles = nt;
        pi.max_row_tiles = mr;
        pi.max_col_tiles = mc;
    } else {
        // ---- hybrid split: aligned 32x32 tiles with at least HYB_MIN_FILL entries become dense tiles (at most
        // HYB_MAX_ROW_TILES per block row, the fullest first), everything else stays with the gather kernels
        if (!a->force_element && a->d == 32 && L % 32 == 0 && nnz > 0) {
            constexpr int HYB_MIN_FILL = 128;
            const int nbr = L / 32;
            std::vector<int> t_rp(nbr + 1, 0), t_col, t_row, cnt(nbr);
            std::vector<std::vector<int>> dense_of(nbr);
            long long dense_entries = 0;
            for (int I = 0; I < nbr; ++I) {
                std::fill(cnt.begin(), cnt.end(), 0);
                for (int r = I * 32; r < I * 32 + 32; ++r)
                    for (int k = off[r]; k < off[r + 1]; ++k) cnt[col[k] >> 5]++;
                std::vector<int> cand;
                for (int J = 0; J < nbr; ++J)
                    if (cnt[J] >= HYB_MIN_FILL) cand.push_back(J);
                if ((int)cand.size() > HYB_MAX_ROW_TILES) {
                    std::stable_sort(cand.begin(), cand.end(), [&](int x, int y) { return cnt[x] > cnt[y]; });
                    cand.resize(HYB_MAX_ROW_TILES);
                    std::sort(cand.begin(), cand.end());
                }
                for (int J : cand) {
                    t_col.push_back(J);
                    t_row.push_back(I);
                    dense_entries += cnt[J];
                }
                dense_of[I] = cand;
                t_rp[I + 1] = (int)t_col.size();
            }
            const int nt = (int)t_col.size();
            if (nt > 0 && dense_entries * 2 >= (long long)nnz) {
                std::vector<int> t_pos((size_t)nt * 32, 0), r_off(L + 1, 0), r_col, r_pos;
                std::vector<unsigned> t_bits((size_t)nt * 32, 0u);
                std::vector<int> slot(nbr);
                for (int I = 0; I < nbr; ++I) {
                    std::fill(slot.begin(), slot.end(), -1);
                    for (size_t e = 0; e < dense_of[I].size(); ++e) slot[dense_of[I][e]] = t_rp[I] + (int)e;
                    for (int rr = 0; rr < 32; ++rr) {
                        const int r = I * 32 + rr;
                        for (int k = off[r]; k < off[r + 1]; ++k) {
                            const int t = slot[col[k] >> 5];
                            if (t < 0) {
                                r_col.push_back(col[k]);
                                r_pos.push_back(k);
                            } else {
                                if (!t_bits[(size_t)t * 32 + rr]) t_pos[(size_t)t * 32 + rr] = k;
                                t_bits[(size_t)t * 32 + rr] |= 1u << (col[k] & 31);
                            }
                        }
                        r_off[r + 1] = (int)r_col.size();
                    }
                }
                const int nr = (int)r_col.size();
                // transposed lists: dense tiles by block column, remainder entries column after column
                std::vector<int> t_cp(nbr + 1, 0), t_ct(std::max(nt, 1));
                for (int t = 0; t < nt; ++t) t_cp[t_col[t] + 1]++;
                for (int J = 0; J < nbr; ++J) t_cp[J + 1] += t_cp[J];
                {
                    std::vector<int> fill(t_cp.begin(), t_cp.end() - 1);
                    for (int t = 0; t < nt; ++t) t_ct[fill[t_col[t]]++] = t;
                }
                std::vector<int> t_ci(t_ct.size());
                for (size_t e = 0; e < t_ct.size(); ++e) t_ci[e] = t_row[t_ct[e]];
                std::vector<int> c_ptr(L + 1, 0), c_row(std::max(nr, 1), 0), c_src(std::max(nr, 1), 0);
                for (int e = 0; e < nr; ++e) c_ptr[r_col[e] + 1]++;
                for (int j = 0; j < L; ++j) c_ptr[j + 1] += c_ptr[j];
                {
                    std::vector<int> fill(c_ptr.begin(), c_ptr.end() - 1);
                    for (int i = 0; i < L; ++i)  // rows ascend: every column's entries end up ordered by row
                        for (int e = r_off[i]; e < r_off[i + 1]; ++e) {
                            const int x = fill[r_col[e]]++;
                            c_row[x] = i;
                            c_src[x] = e;
                        }
                }
                if (r_col.empty()) {
                    r_col.push_back(0);
                    r_pos.push_back(0);
                }
                std::vector<int> bits_as_int(t_bits.size());
                memcpy(bits_as_int.data(), t_bits.data(), t_bits.size() * sizeof(int));
                hyb_off[0] = append(t_rp);
                hyb_off[1] = append(t_col);
                hyb_off[3] = append(t_pos);
                hyb_off[4] = append(bits_as_int);
                hyb_off[5] = append(t_cp);
                hyb_off[6] = append(t_ct);
                hyb_off[7] = append(r_off);
                hyb_off[8] = append(r_col);
                hyb_off[9] = append(r_pos);
                hyb_off[10] = append(c_ptr);
                hyb_off[11] = append(c_row);
                hyb_off[12] = append(c_src);
                hyb_off[13] = append(t_ci);
                pi.hyb_nr = nr;
                pi.hybrid = true;
                pi.hyb_tiles = nt;
                for (int I = 0; I < nbr; ++I) {
                    pi.max_row_tiles = std::max(pi.max_row_tiles, t_rp[I + 1] - t_rp[I]);
                    pi.max_col_tiles = std::max(pi.max_col_tiles, t_cp[I + 1] - t_cp[I]);
                }
            }
        }
        std::vector<int> ccp(L + 1, 0), crow(std::max(nnz, 1)), cpos(std::max(nnz, 1));
        for (int k = 0; k < nnz; ++k) ccp[col[k] + 1]++;
        for (int j = 0; j < L; ++j) ccp[j + 1] += ccp[j];
        std::vector<int> fill(ccp.begin(), ccp.end() - 1);
        for (int i = 0; i < L; ++i)
            for (int k = off[i]; k < off[i + 1]; ++k) {
                int e = fill[col[k]]++;
                crow[e] = i;
                cpos[e] = k;
            }
        o_ccp = append(ccp);
        o_crow = append(crow);
        o_cpos = append(cpos);
    }
    if (!SPION_HIP_OK(hipMalloc((void**)&pi.d_blob, sizeof(int) * blob.size()))) return false;
    if (!SPION_HIP_OK(hipMemcpy(pi.d_blob, blob.data(), sizeof(int) * blob.size(), hipMemcpyHostToDevice))) {
        pi.release();
        return false;
    }
    if (tiled) {
        pi.d_trp = pi.d_blob + o_trp;
        pi.d_tcol = pi.d_blob + o_tcol;
        pi.d_tcp = pi.d_blob + o_tcp;
        pi.d_tcdesc = pi.d_blob + o_tcdesc;
        pi.d_rdesc = pi.d_blob + o_rdesc;
        pi.d_fdesc = pi.d_blob + o_fdesc;
        pi.d_cdesc = pi.d_blob + o_cdesc;
        Bf16Plan* plans[3] = {&pi.plan_row, &pi.plan_pair, &pi.plan_col};
        for (int k = 0; k < 3; ++k)
            if (plans[k]->lanes) {
                plans[k]->sched = Bf16Sched{pi.d_blob + o_plan[k][0], pi.d_blob + o_plan[k][1], pi.d_blob + o_plan[k][2]};
                plans[k]->d_longs = pi.d_blob + o_plan[k][3];
            }
    } else {
        pi.d_ccp = pi.d_blob + o_ccp;
        pi.d_crow = pi.d_blob + o_crow;
        pi.d_cpos = pi.d_blob + o_cpos;
        if (pi.hybrid) {
            const int* b = pi.d_blob;
            pi.hyb = HybIndex{b + hyb_off[0], b + hyb_off[1], b + hyb_off[3],
                              reinterpret_cast<const unsigned*>(b + hyb_off[4]), b + hyb_off[5], b + hyb_off[6],
                              b + hyb_off[13], b + hyb_off[7], b + hyb_off[8], b + hyb_off[9], b + hyb_off[10],
                              b + hyb_off[11], b + hyb_off[12], pi.hyb_nr, pi.hyb_tiles};
        }
    }
    pi.tiled = tiled;
    pi.key_off = Offsets;
    pi.key_col = Columns;
    pi.key_nnz = nnz;
    pi.valid = true;
    // install: the slot already filed under this key (re-registration), else a free one, else the least recently used
    int slot = -1;
    for (int i = 0; i < SparseAttn::PAT_SLOTS; ++i)
        if (a->pats[i].valid && a->pats[i].key_off == Offsets && a->pats[i].key_col == Columns) slot = i;
    for (int i = 0; i < SparseAttn::PAT_SLOTS && slot < 0; ++i)
        if (!a->pats[i].valid) slot = i;
    if (slot < 0) {
        slot = 0;
        for (int i = 1; i < SparseAttn::PAT_SLOTS; ++i)
            if (a->pat_stamp[i] < a->pat_stamp[slot]) slot = i;
    }
    a->pats[slot].release();  // hipFree waits for the kernels that may still read the evicted index
    a->pats[slot] = pi;
    a->pat_stamp[slot] = ++a->pat_clock;
    a->pat = pi;
    return true;
}

static bool ensure_pattern(SparseAttn* a, const int* Offsets, const int* Columns, int nnz) {
    const PatternIndex& cur = a->pat;
    if (cur.valid && cur.key_off == Offsets && cur.key_col == Columns && cur.key_nnz == nnz) return true;
    for (int i = 0; i < SparseAttn::PAT_SLOTS; ++i) {
        const PatternIndex& pi = a->pats[i];
        if (pi.valid && pi.key_off == Offsets && pi.key_col == Columns && pi.key_nnz == nnz) {
            a->pat_stamp[i] = ++a->pat_clock;
            a->pat = pi;
            return true;
        }
    }
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(a->hdr.stream, &cap);
    if (cap != hipStreamCaptureStatusNone) {
        set_error("pattern: an index that was never analysed cannot be analysed while its stream is being captured "
                  "(run the call once before the capture, or register the pattern)");
        return false;
    }
    return analyse_pattern(a, Offsets, Columns, nnz);
}

// Analyse a pattern from host copies of its index arrays and file it under the device arrays' key: the first
// forward then copies nothing back and does not wait for the stream.
int sparse_register_pattern(void* h, const int* Offsets, const int* Columns, int nnz, const int* host_off,
                            const int* host_col) {
    SparseAttn* a = as_sparse(h, "spion_register_pattern");
    if (!a) return 1;
    if (!Offsets || !host_off || (nnz > 0 && (!Columns || !host_col))) {
        set_error("spion_register_pattern: null pointer argument");
        return 1;
    }
    return analyse_pattern(a, Offsets, Columns, nnz, host_off, host_col) ? 0 : 1;
}

// Drop the analysis filed under (Offsets, Columns), if any.
void sparse_forget_pattern(void* h, const int* Offsets, const int* Columns) {
    SparseAttn* a = as_sparse(h, "spion_forget_pattern");
    if (!a) return;
    for (auto& pi : a->pats)
        if (pi.valid && pi.key_off == Offsets && pi.key_col == Columns) pi.release();
    if (a->pat.valid && a->pat.key_off == Offsets && a->pat.key_col == Columns) a->pat = PatternIndex();
}

static bool ensure_ws(float** p, size_t count) {
    if (*p) return true;
    return SPION_HIP_OK(hipMalloc((void**)p, sizeof(float) * count));
}

// A workspace whose size follows the pattern: grown (never under HIP graph capture, where an allocation would
// invalidate the capture) to at least the size asked for, by half of its size or more so that a series of slightly
// larger patterns does not allocate every time.  The buffer it replaces is not freed but retired until the handle
// is destroyed: a graph recorded before the growth keeps working on the old buffer, which is large enough for the
// pattern it was recorded with.
static bool ensure_ws_grow(SparseAttn* a, float** p, size_t* have, size_t need, const char* who) {
    if (*have >= need) return true;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(a->hdr.stream, &cap);
    if (cap != hipStreamCaptureStatusNone) {
        set_error("%s: the workspace for this pattern is not allocated yet; run one step outside the capture", who);
        return false;
    }
    const size_t want = std::max(need, *have + *have / 2);
    float* fresh = nullptr;
    if (hipMalloc((void**)&fresh, sizeof(float) * want) != hipSuccess) {
        (void)hipGetLastError();
        if (want == need || !SPION_HIP_OK(hipMalloc((void**)&fresh, sizeof(float) * need))) {
            if (want == need) set_error("%s: hipMalloc of %zu bytes of workspace failed", who, sizeof(float) * need);
            return false;
        }
        *have = need;
    } else {
        *have = want;
    }
    if (*p) a->retired.push_back(*p);
    *p = fresh;
    return true;
}

int transpose_last2(const float* in, float* out, int batch, int rows, int cols, hipStream_t stream);

// Slot of the O copy for the forward that fills P buffer `key` (least recently used slot on a miss).
static float* ocache_for_forward(SparseAttn* a, const float* key) {
    if (!a->use_ocache) return nullptr;
    SparseAttn::OSlot* pick = nullptr;
    for (auto& sl : a->oslot)
        if (sl.key == key) pick = &sl;
    if (!pick) {
        pick = &a->oslot[0];
        for (auto& sl : a->oslot)
            if (sl.stamp < pick->stamp) pick = &sl;
    }
    if (!pick->buf) {
        // All slots are allocated on the first forward, so that later calls -- under HIP graph capture, where an
        // allocation would invalidate the capture -- find a buffer whatever P pointer they are handed.
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        (void)hipStreamIsCapturing(a->hdr.stream, &cap);
        if (cap == hipStreamCaptureStatusNone)
            for (auto& sl : a->oslot)
                if (!sl.buf && hipMalloc((void**)&sl.buf, sizeof(float) * (size_t)a->NB * a->L * a->d) != hipSuccess) {
                    (void)hipGetLastError();
                    sl.buf = nullptr;
                    break;
                }
        if (!pick->buf) {  // no copy: the backward falls back to the two-sweep kernel
            pick->key = nullptr;
            return nullptr;
        }
    }
    pick->key = key;
    pick->stamp = ++a->ostamp;
    return pick->buf;
}
// A forward that fills P buffer `key` without refreshing a kept copy of O (strided heads, element kernels) must
// not leave an older copy filed under that pointer: a later backward handed the same P would take its row sums
// from it.
static void ocache_drop(SparseAttn* a, const float* key) {
    for (auto& sl : a->oslot)
        if (sl.key == key) sl.key = nullptr;
}
static const float* ocache_for_backward(SparseAttn* a, const float* key) {
    if (!a->use_ocache) return nullptr;
    for (auto& sl : a->oslot)
        if (sl.key == key && sl.buf) return sl.buf;
    return nullptr;
}

// Wavefronts per strip (block row or block column).  Forward: enough waves that each one's share of the
// longest block row stays in registers (8 logit tiles at d = 32, 4 at d = 64).  Backward: one wave per strip
// -- no cross-wave merge and the longest software pipeline -- unless strips are long and the launch is
// too small to fill the 1024 SIMDs with single-wave work-groups.
static int pick_waves(const SparseAttn* a, const PatternIndex& pi, int nbr, bool forward) {
    const int avg = nbr ? (pi.ntiles + nbr - 1) / nbr : 0;
    const long long strips = (long long)nbr * a->NB;
    if (forward) {
        const int maxt = a->d == 32 ? 8 : 4;
        const int fit = pi.max_row_tiles <= maxt ? 1 : pi.max_row_tiles <= 2 * maxt ? 2 : 4;
        // A launch that fills the machine anyway takes the fewest waves that keep the logits in registers: no
        // cross-wave merge and more tiles per wave (measured at L = 1024, 4.3 tiles per row on average:
        // 0.18 ms with one wave against 0.25 ms with four at 16384 rows, a tie at 1024 rows, the reverse at 512).
        if (strips >= 2048) return fit;
        if (strips >= 1024) return std::max(fit, 2);
        if (pi.max_row_tiles <= maxt && avg <= 2) return 1;
        if (pi.max_row_tiles <= 2 * maxt && avg <= 4) return 2;
        return 4;
    }
    // a few very long strips (global rows / columns) would leave one wave working alone at the end
    if (std::max(pi.max_row_tiles, pi.max_col_tiles) > 8 * avg + 16) return 4;
    if (strips >= 2048 || avg <= 2) return 1;
    if (strips >= 1024 || avg <= 4) return 2;
    return 4;
}

// Heads whose strips are interleaved in launch order (see item_to_head_strip).
static int heads_per_group(const SparseAttn* a) {
    // Two heads share a stretch of the launch order when every die's share of the heads is even: the long strips of
    // both come first, so the last work groups of a die are short ones (north star shape: step 2 % shorter than
    // with one head at a time; four heads give the same, eight lose it again to the L2's reach).
    return a->NB % 16 == 0 ? 2 : 1;
}

template <int D, bool MASK, bool KROW, bool ST = false>
static void launch_tile_fwd(SparseAttn* a, const float* Q, const float* Kt, const float* V, const float* pen, float* P,
                            float* O, const int* offs, int nnz, const Layouts& ly = Layouts{}) {
    PhaseRange phase("spion forward (tile kernels)");
    const PatternIndex& pi = a->pat;
    const int nbr = a->L / 32;
    float* ocache = ST ? nullptr : ocache_for_forward(a, P);
    if (!ocache) ocache_drop(a, P);
    // Logit tiles stay in registers when every wavefront's share of the longest block row fits (MAXT tiles);
    // otherwise two sweeps.  (Launching the block rows by length class with 1, 2 and 4 wavefronts per row was
    // measured and brings nothing over four wavefronts for all.)
    constexpr int MAXT = D == 32 ? 8 : 4;
    const int wv = pick_waves(a, pi, nbr, true);
    const int hc = heads_per_group(a);
    // d = 32, four wavefronts per strip: the strips of at most 16 tiles (four per wavefront) run three work-groups
    // to a CU in a launch of their own, the few longer ones first with eight tiles per wavefront (north star:
    // forward 0.1756 -> 0.1721 ms; six wavefronts of four tiles for the long strips instead: 44 against 36 us)
    static const bool no_split = getenv("SPION_NO_FWD_SPLIT") != nullptr;
    // A pattern with a few strips far longer than the rest (global rows): those, and whatever else exceeds 24 tiles,
    // take the two sweeps with eight wavefronts to a strip in a launch of their own, which goes first on the caller's
    // stream; all other strips follow on the handle's side stream with six logit tiles per wavefront (see
    // launch_tile_bwd for the streams).
    static const bool no_long = getenv("SPION_NO_LONG_SPLIT") != nullptr;
    const int n24 = pi.n_fwd_long24;
    if (!no_long && a->side && wv == 4 && pi.n_long_rows > 0 && n24 * 8 <= nbr) {
        (void)hipEventRecord(a->side_fork, a->hdr.stream);
        (void)hipStreamWaitEvent(a->side, a->side_fork, 0);
        hipLaunchKernelGGL((tile_fwd_kernel<D, 8, MASK, 0, KROW, ST>), dim3(n24 * a->NB), dim3(512), 0, a->hdr.stream, Q,
                           Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr, a->NB, nnz, a->scale, 0, n24, hc, ly);
        hipLaunchKernelGGL((tile_fwd_kernel<D, 4, MASK, 6, KROW, ST>), dim3((nbr - n24) * a->NB), dim3(256), 0, a->side,
                           Q, Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr, a->NB, nnz, a->scale, n24,
                           nbr - n24, hc, ly);
        (void)hipEventRecord(a->side_join, a->side);
        (void)hipStreamWaitEvent(a->hdr.stream, a->side_join, 0);
        return;
    }
    if constexpr (D == 32) {
        // longest strip of 17 to 24 tiles: six logit tiles per wavefront still fit three work-groups to a CU (161
        // registers), so one launch takes every strip (north star: forward 0.171 -> 0.166 ms against the split)
        if (wv == 4 && pi.max_row_tiles <= 24 && pi.max_row_tiles > 16) {
            hipLaunchKernelGGL((tile_fwd_kernel<D, 4, MASK, 6, KROW, ST>), dim3(nbr * a->NB), dim3(256), 0, a->hdr.stream,
                               Q, Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr, a->NB, nnz, a->scale, 0, nbr,
                               hc, ly);
            return;
        }
        // a few strips of more than 32 tiles (global rows) among strips of at most 24: the six-tile kernel with the two
        // sweeps for the long ones inside the same launch, instead of the two sweeps for every strip
        if (wv == 4 && pi.max_row_tiles > 4 * MAXT && pi.n_fwd_long24 * 4 < nbr) {
            hipLaunchKernelGGL((tile_fwd_kernel<D, 4, MASK, 6, KROW, ST, true>), dim3(nbr * a->NB), dim3(256), 0,
                               a->hdr.stream, Q, Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr, a->NB, nnz,
                               a->scale, 0, nbr, hc, ly);
            return;
        }
        if (wv == 4 && !no_split && pi.max_row_tiles <= 4 * MAXT && pi.n_fwd_long < nbr && pi.max_row_tiles > 16) {
            const int nl = pi.n_fwd_long;
            if (nl > 0)
                hipLaunchKernelGGL((tile_fwd_kernel<D, 4, MASK, MAXT, KROW, ST>), dim3(nl * a->NB), dim3(256), 0,
                                   a->hdr.stream, Q, Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr, a->NB,
                                   nnz, a->scale, 0, nl, hc, ly);
            hipLaunchKernelGGL((tile_fwd_kernel<D, 4, MASK, 4, KROW, ST>), dim3((nbr - nl) * a->NB), dim3(256), 0,
                               a->hdr.stream, Q, Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr, a->NB, nnz,
                               a->scale, nl, nbr - nl, hc, ly);
            return;
        }
    }
    if constexpr (D == 64) {
        // most strips of at most 24 tiles, a few longer ones: six logit tiles per wavefront, and the long strips take
        // the two sweeps inside the same launch
        if (wv == 4 && pi.max_row_tiles > 4 * MAXT && pi.n_fwd_long24 * 4 < nbr) {
            hipLaunchKernelGGL((tile_fwd_kernel<D, 4, MASK, 6, KROW, ST>), dim3(nbr * a->NB), dim3(256), 0, a->hdr.stream,
                               Q, Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr, a->NB, nnz, a->scale, 0, nbr,
                               hc, ly);
            return;
        }
    }
#define SPION_LAUNCH(W)                                                                                              \
    do {                                                                                                             \
        if (pi.max_row_tiles <= W * MAXT)                                                                            \
            hipLaunchKernelGGL((tile_fwd_kernel<D, W, MASK, MAXT, KROW, ST>), dim3(nbr * a->NB), dim3(64 * W), 0,        \
                               a->hdr.stream, Q, Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr,     \
                               a->NB, nnz, a->scale, 0, nbr, hc, ly);                                                    \
        else                                                                                                         \
            hipLaunchKernelGGL((tile_fwd_kernel<D, W, MASK, 0, KROW, ST>), dim3(nbr * a->NB), dim3(64 * W), 0,           \
                               a->hdr.stream, Q, Kt, V, pen, P, O, ocache, pi.d_fdesc, pi.d_tcol, a->L, nbr,     \
                               a->NB, nnz, a->scale, 0, nbr, hc, ly);                                                    \
    } while (0)
    if (wv == 1) SPION_LAUNCH(1);
    else if (wv == 2) SPION_LAUNCH(2);
    else SPION_LAUNCH(4);
#undef SPION_LAUNCH
}

// One launch of a backward pass over the strips s0 .. s0+ns-1 of every head's strip order, W wavefronts per strip.
template <int D, int W, bool VROW, bool ST>
static void launch_tile_bwd_rows(SparseAttn* a, hipStream_t stream, const float* K, const float* Vt, const float* P,
                                 const float* dO, const float* ocache, float* rowsum, float* dQ, int nnz, int hc,
                                 const Layouts& ly, int s0, int ns) {
    const PatternIndex& pi = a->pat;
    const int nbr = a->L / 32;
    const dim3 grid(ns * a->NB), block(64 * W);
    if (ocache) {
        hipLaunchKernelGGL((tile_bwd_row_kernel<D, W, true, VROW, ST>), grid, block, 0, stream, K, Vt, P, dO, ocache,
                           rowsum, dQ, pi.d_rdesc, pi.d_tcol, a->L, nbr, a->NB, nnz, a->scale, hc, ly, s0, ns);
    } else {
        if constexpr (!ST)
            hipLaunchKernelGGL((tile_bwd_row_kernel<D, W, false, VROW>), grid, block, 0, stream, K, Vt, P, dO, ocache,
                               rowsum, dQ, pi.d_rdesc, pi.d_tcol, a->L, nbr, a->NB, nnz, a->scale, hc, ly, s0, ns);
    }
}
template <int D, int W, bool VROW, bool ST>
static void launch_tile_bwd_cols(SparseAttn* a, hipStream_t stream, const float* Q, const float* Vt, const float* P,
                                 const float* dO, const float* rowsum, float* dK, float* dV, int nnz, int hc,
                                 const Layouts& ly, int s0, int ns) {
    const PatternIndex& pi = a->pat;
    const int nbr = a->L / 32;
    hipLaunchKernelGGL((tile_bwd_col_kernel<D, W, VROW, ST>), dim3(ns * a->NB), dim3(64 * W), 0, stream, Q, Vt, P, dO,
                       rowsum, dK, dV, pi.d_cdesc, pi.d_tcdesc, a->L, nbr, a->NB, nnz, a->scale, hc, ly, s0, ns);
}

// Wavefronts per strip of a backward launch over strips of at most `longest` tiles.
static int bwd_waves(const SparseAttn* a, const PatternIndex& pi, int nbr, int strips_per_head) {
    const int avg = nbr ? (pi.ntiles + nbr - 1) / nbr : 0;
    const long long strips = (long long)strips_per_head * a->NB;
    if (strips >= 2048 || avg <= 2) return 1;
    if (strips >= 1024 || avg <= 4) return 2;
    return 4;
}

template <int D, bool VROW, bool ST = false>
static void launch_tile_bwd(SparseAttn* a, const float* Q, const float* K, const float* Vt, const float* P,
                            const float* dO, float* dQ, float* dK, float* dV, const int* offs, int nnz,
                            const float* Out, const Layouts& ly = Layouts{}, float* rowsum = nullptr) {
    const PatternIndex& pi = a->pat;
    // the entry point that allocates nothing brings its own row-sum array and creates nothing either
    const bool side_ok = rowsum == nullptr;
    if (!rowsum) rowsum = a->ws_rowsum;
    const int nbr = a->L / 32;
    const int hc = heads_per_group(a);
    const float* ocache = Out ? Out : ocache_for_backward(a, P);
    // A pattern with a few strips far longer than the rest (global rows, global columns): those run four wavefronts
    // to a strip in a small launch of their own, all other strips in a launch with the wavefront count their own
    // number calls for -- instead of four wavefronts to every strip of the pattern because of the few.  The large
    // launch goes to a side stream of the handle (made when such a pattern is analysed), beside the small one; without
    // that stream the two launches follow one another, with the same results.
    static const bool no_split = getenv("SPION_NO_LONG_SPLIT") != nullptr;
    const int nlr = pi.n_long_rows, nlc = pi.n_long_cols;
    const bool split = !no_split && (nlr > 0 || nlc > 0) && nlr * 8 <= nbr && nlc * 8 <= nbr;
    const bool side = split && side_ok && a->side != nullptr;
    // the long strips go first, on the caller's stream, so that they hold their places on the CUs before the many
    // short work-groups arrive; those follow on the side stream
    hipStream_t rest_stream = side ? a->side : a->hdr.stream;
    auto fork = [&]() {
        if (!side) return;
        (void)hipEventRecord(a->side_fork, a->hdr.stream);
        (void)hipStreamWaitEvent(a->side, a->side_fork, 0);
    };
    auto join = [&]() {
        if (!side) return;
        (void)hipEventRecord(a->side_join, a->side);
        (void)hipStreamWaitEvent(a->hdr.stream, a->side_join, 0);
    };
#define SPION_ROWS(W, STREAM, S0, NS) \
    launch_tile_bwd_rows<D, W, VROW, ST>(a, STREAM, K, Vt, P, dO, ocache, rowsum, dQ, nnz, hc, ly, S0, NS)
#define SPION_COLS(W, STREAM, S0, NS) \
    launch_tile_bwd_cols<D, W, VROW, ST>(a, STREAM, Q, Vt, P, dO, rowsum, dK, dV, nnz, hc, ly, S0, NS)
#define SPION_BY_WAVES(WV, WHAT, STREAM, S0, NS)      \
    do {                                              \
        if ((WV) == 1) WHAT(1, STREAM, S0, NS);       \
        else if ((WV) == 2) WHAT(2, STREAM, S0, NS);  \
        else WHAT(4, STREAM, S0, NS);                 \
    } while (0)
    if (split) {
        if (a->bwd_passes & 1) {
            PhaseRange range("spion backward: row pass (dQ)");
            const int wv = bwd_waves(a, pi, nbr, nbr - nlr);
            if (nlr > 0) {
                fork();
                SPION_ROWS(8, a->hdr.stream, 0, nlr);
            }
            SPION_BY_WAVES(wv, SPION_ROWS, nlr > 0 ? rest_stream : a->hdr.stream, nlr, nbr - nlr);
            if (nlr > 0) join();
        }
        if (a->bwd_passes & 2) {
            PhaseRange range("spion backward: column pass (dK, dV)");
            const int wv = bwd_waves(a, pi, nbr, nbr - nlc);
            if (nlc > 0) {
                fork();
                SPION_COLS(8, a->hdr.stream, 0, nlc);
            }
            SPION_BY_WAVES(wv, SPION_COLS, nlc > 0 ? rest_stream : a->hdr.stream, nlc, nbr - nlc);
            if (nlc > 0) join();
        }
    } else {
        const int wv = pick_waves(a, pi, nbr, false);
        if (a->bwd_passes & 1) {
            PhaseRange range("spion backward: row pass (dQ)");
            SPION_BY_WAVES(wv, SPION_ROWS, a->hdr.stream, 0, nbr);
        }
        if (a->bwd_passes & 2) {
            PhaseRange range("spion backward: column pass (dK, dV)");
            SPION_BY_WAVES(wv, SPION_COLS, a->hdr.stream, 0, nbr);
        }
    }
#undef SPION_ROWS
#undef SPION_COLS
#undef SPION_BY_WAVES
}

// The remainder's column pass with its gathered operands in LDS: columns per lane group (work-groups of 1024, 512 or
// 256 columns of a head), the most that still gives every CU a work-group -- with half of them idle the kernel that
// gathers from L2 is as fast (configuration 4 at half its batch: 0.248 against 0.244 ms) -- or 0 for that kernel
// (also with SPION_HYB_GATHER=1).
static int hyb_lds_columns(const SparseAttn* a) {
    static const bool gather = getenv("SPION_HYB_GATHER") != nullptr;
    if (gather || a->L % 1024) return 0;
    for (int nc = 8; nc >= 2; nc >>= 1)
        if ((long long)a->NB * (a->L / (128 * nc)) >= 256) return nc;
    return 0;
}
// The same for the forward's logits of the remainder: work-groups of 512 rows (four per lane group; eight need more
// registers than a wavefront of sixteen has and are no faster), when every CU gets one.
static bool hyb_lds_rows(const SparseAttn* a) {
    static const bool gather = getenv("SPION_HYB_GATHER") != nullptr;
    return !gather && a->L % 1024 == 0 && (long long)a->NB * (a->L / 512) >= 256;
}
#define SPION_HYB_COL_LDS(ST_, PAIRS_, NC_, ...)                                                          \
    hipLaunchKernelGGL((hyb_rem_bwd_col_lds_kernel<ST_, PAIRS_, NC_>), dim3(a->NB * (a->L / (128 * NC_))), \
                       dim3(HYB_CL_THREADS), 0, a->hdr.stream, __VA_ARGS__)

// Hybrid patterns (dense tiles + remainder, d = 32).  Every operand row-major; ST: heads located by `ly`.
// ocopy (contiguous heads only): where a second copy of O goes, or null.
template <bool ST>
static void launch_hyb_fwd(SparseAttn* a, const float* Q, const float* K, const float* V, const float* Mask,
                           float* Attn, float* Out, float* ocopy, const int* Offsets, int nnz, const Layouts& ly) {
    PhaseRange phase("spion forward (hybrid kernels)");
    if (!ensure_ws(&a->ws_stats, (size_t)a->NB * a->L * 2)) return;
    // the remainder's raw logits between the first and the third launch: a compact list of their own (written and
    // read in full lines) rather than their places inside P, where every four-byte store would pull in a line
    if (!ensure_ws_grow(a, &a->ws_raw, &a->ws_raw_count, (size_t)a->NB * (size_t)std::max(a->pat.hyb_nr, 1),
                        "attn_forward"))
        return;
    a->last_path = 3;
    const int nbr = a->L / 32;
    const long long rows = (long long)a->NB * a->L;
    // strips of few dense tiles: one wavefront walks the whole strip; else four share it
    const bool one = a->pat.max_row_tiles <= HYB_MAXT1;
    const dim3 grid_t(nbr * a->NB), block_t(one ? 64 : 256);
    const dim3 grid_g((unsigned)((rows + HYB_GWAVES - 1) / HYB_GWAVES)), block_g(64 * HYB_GWAVES);
    float2* stats = reinterpret_cast<float2*>(a->ws_stats);
    const bool lds_logits = hyb_lds_rows(a);
#define SPION_HYB_LOGITS_LDS(MASKED, NR_)                                                                            \
    hipLaunchKernelGGL((hyb_rem_logits_lds_kernel<MASKED, ST, NR_>), dim3(a->NB * (a->L / (128 * NR_))),             \
                       dim3(HYB_LL_THREADS), 0, a->hdr.stream, Q, K, Mask, a->ws_raw, stats, a->pat.hyb, a->L, a->NB, \
                       a->scale, ly)
#define SPION_HYB_FWD(MASKED)                                                                                        \
    do {                                                                                                             \
        if (lds_logits) SPION_HYB_LOGITS_LDS(MASKED, 4);                                                             \
        else                                                                                                         \
        hipLaunchKernelGGL((hyb_rem_logits_kernel<MASKED, ST>), grid_g, block_g, 0, a->hdr.stream, Q, K, Mask,       \
                           a->ws_raw, stats, a->pat.hyb, a->L, a->NB, a->scale, ly);                                 \
        if (one)                                                                                                     \
            hipLaunchKernelGGL((hyb_tile_fwd_kernel<MASKED, 1, HYB_MAXT1, ST>), grid_t, block_t, 0, a->hdr.stream,   \
                               Q, K, V, Mask, Attn, Out, stats, Offsets, a->pat.hyb, a->L, nbr, a->NB, nnz,          \
                               a->scale, ly);                                                                        \
        else                                                                                                         \
            hipLaunchKernelGGL((hyb_tile_fwd_kernel<MASKED, 4, HYB_MAXT4, ST>), grid_t, block_t, 0, a->hdr.stream,   \
                               Q, K, V, Mask, Attn, Out, stats, Offsets, a->pat.hyb, a->L, nbr, a->NB, nnz,          \
                               a->scale, ly);                                                                        \
    } while (0)
    if (a->has_mask)
        SPION_HYB_FWD(true);
    else
        SPION_HYB_FWD(false);
#undef SPION_HYB_FWD
#undef SPION_HYB_LOGITS_LDS
    if (hyb_lds_columns(a) == 8)  // a full machine of work-groups of 1024 rows: the V rows in LDS
        hipLaunchKernelGGL(hyb_rem_pv_lds_kernel<ST>, dim3(a->NB * (a->L / HYB_RL_ROWS)), dim3(HYB_RL_THREADS), 0,
                           a->hdr.stream, V, (const float*)a->ws_raw, Attn, Out, ocopy, (const float2*)stats, a->pat.hyb,
                           a->L, a->NB, nnz, ly);
    else
        hipLaunchKernelGGL(hyb_rem_pv_kernel<ST>, grid_g, block_g, 0, a->hdr.stream, V, (const float*)a->ws_raw, Attn,
                           Out, ocopy, (const float2*)stats, a->pat.hyb, a->L, a->NB, nnz, ly);
    check_launch("hybrid forward kernels");
}

// o: the forward's output (same layout as dO).  dS: the caller's [NB][nnz] scratch, which receives the remainder's
// {dS, P} pairs, [NB][nr] (a hybrid pattern keeps at most half of its entries in the remainder).
template <bool ST>
static void launch_hyb_bwd(SparseAttn* a, const float* Q, const float* K, const float* V, const float* P,
                           const float* dO, const float* o, float* dS, float* dQ, float* dK, float* dV, int nnz,
                           const Layouts& ly) {
    PhaseRange phase("spion backward (hybrid kernels)");
    if (!ensure_ws(&a->ws_rowsum, (size_t)a->NB * a->L)) return;
    a->last_path = 3;
    const int nbr = a->L / 32;
    const long long rows = (long long)a->NB * a->L;
    const bool one_r = a->pat.max_row_tiles <= 2 * HYB_MAXT1, one_c = a->pat.max_col_tiles <= 2 * HYB_MAXT1;
    const dim3 grid_t(nbr * a->NB);
    const dim3 grid_g((unsigned)((rows + HYB_GWAVES - 1) / HYB_GWAVES)), block_g(64 * HYB_GWAVES);
    float2* pairs = reinterpret_cast<float2*>(dS);
    if (a->bwd_passes & 1) {
        if (one_r)
            hipLaunchKernelGGL((hyb_tile_bwd_row_kernel<1, ST>), grid_t, dim3(64), 0, a->hdr.stream, K, V, P, dO, o,
                               a->ws_rowsum, dQ, a->pat.hyb, a->L, nbr, a->NB, nnz, a->scale, ly);
        else
            hipLaunchKernelGGL((hyb_tile_bwd_row_kernel<4, ST>), grid_t, dim3(256), 0, a->hdr.stream, K, V, P, dO, o,
                               a->ws_rowsum, dQ, a->pat.hyb, a->L, nbr, a->NB, nnz, a->scale, ly);
        hipLaunchKernelGGL(hyb_rem_bwd_row_kernel<ST>, grid_g, block_g, 0, a->hdr.stream, K, V, P, dO,
                           (const float*)a->ws_rowsum, pairs, dQ, a->pat.hyb, a->L, a->NB, nnz, a->scale, ly);
    }
    if (a->bwd_passes & 2) {
        if (one_c)
            hipLaunchKernelGGL((hyb_tile_bwd_col_kernel<1, ST>), grid_t, dim3(64), 0, a->hdr.stream, Q, V, P, dO,
                               (const float*)a->ws_rowsum, dK, dV, a->pat.hyb, a->L, nbr, a->NB, nnz, a->scale, ly);
        else
            hipLaunchKernelGGL((hyb_tile_bwd_col_kernel<4, ST>), grid_t, dim3(256), 0, a->hdr.stream, Q, V, P, dO,
                               (const float*)a->ws_rowsum, dK, dV, a->pat.hyb, a->L, nbr, a->NB, nnz, a->scale, ly);
        const int nc = hyb_lds_columns(a);
        if (nc == 8)
            SPION_HYB_COL_LDS(ST, true, 8, Q, dO, (const float2*)pairs, nullptr, nullptr, dK, dV, a->pat.hyb.c_ptr,
                              a->pat.hyb.c_row, a->pat.hyb.c_src, a->pat.hyb.nr, a->L, a->NB, ly);
        else if (nc == 4)
            SPION_HYB_COL_LDS(ST, true, 4, Q, dO, (const float2*)pairs, nullptr, nullptr, dK, dV, a->pat.hyb.c_ptr,
                              a->pat.hyb.c_row, a->pat.hyb.c_src, a->pat.hyb.nr, a->L, a->NB, ly);
        else if (nc == 2)
            SPION_HYB_COL_LDS(ST, true, 2, Q, dO, (const float2*)pairs, nullptr, nullptr, dK, dV, a->pat.hyb.c_ptr,
                              a->pat.hyb.c_row, a->pat.hyb.c_src, a->pat.hyb.nr, a->L, a->NB, ly);
        else
            hipLaunchKernelGGL(hyb_rem_bwd_col_kernel<ST>, grid_g, block_g, 0, a->hdr.stream, Q, dO,
                               (const float2*)pairs, dK, dV, a->pat.hyb, a->L, a->NB, ly);
    }
    check_launch("hyb_bwd kernels");
}

static void launch_transpose(SparseAttn* a, const float* Xt, float* X) {
    dim3 grid((a->L + 31) / 32, (a->d + 31) / 32, a->NB);
    hipLaunchKernelGGL(transpose_dl_kernel, grid, dim3(256), 0, a->hdr.stream, Xt, X, a->d, a->L);
}

template <int D, bool ST = false>
static void launch_elem_fwd(SparseAttn* a, const float* Q, const float* Krm, const float* V, const float* pen,
                            float* P, float* O, const int* offs, const int* cols, int nnz,
                            const Layouts& ly = Layouts{}) {
    PhaseRange phase("spion forward (element kernels)");
    const long long rows = (long long)a->NB * a->L;
    dim3 grid((unsigned)((rows + ELEM_WAVES - 1) / ELEM_WAVES));
    if (a->has_mask)
        hipLaunchKernelGGL((elem_fwd_kernel<D, true, ST>), grid, dim3(64 * ELEM_WAVES), 0, a->hdr.stream, Q, Krm, V,
                           pen, P, O, offs, cols, a->L, a->NB, nnz, a->scale, ly);
    else
        hipLaunchKernelGGL((elem_fwd_kernel<D, false, ST>), grid, dim3(64 * ELEM_WAVES), 0, a->hdr.stream, Q, Krm, V,
                           pen, P, O, offs, cols, a->L, a->NB, nnz, a->scale, ly);
}

template <int D, bool ST = false>
static void launch_elem_bwd(SparseAttn* a, const float* Q, const float* K, const float* Vrm, const float* P,
                            const float* dO, float* dS, float* dQ, float* dK, float* dV, const int* offs,
                            const int* cols, int nnz, const Layouts& ly = Layouts{}) {
    PhaseRange phase("spion backward (element kernels)");
    const PatternIndex& pi = a->pat;
    const long long rows = (long long)a->NB * a->L;
    dim3 grid((unsigned)((rows + ELEM_WAVES - 1) / ELEM_WAVES));
    if (a->bwd_passes & 1)
        hipLaunchKernelGGL((elem_bwd_row_kernel<D, ST>), grid, dim3(64 * ELEM_WAVES), 0, a->hdr.stream, K, Vrm, P, dO,
                           dS, dQ, offs, cols, a->L, a->NB, nnz, a->scale, ly);
    if (a->bwd_passes & 2) {
        if constexpr (D == 32) {
            const int nc = hyb_lds_columns(a);  // the Q and dO rows of a range of the sequence in LDS, see hybrid_kernels.h
            if (nc == 8)
                SPION_HYB_COL_LDS(ST, false, 8, Q, dO, nullptr, dS, P, dK, dV, pi.d_ccp, pi.d_crow, pi.d_cpos, nnz, a->L,
                                  a->NB, ly);
            else if (nc == 4)
                SPION_HYB_COL_LDS(ST, false, 4, Q, dO, nullptr, dS, P, dK, dV, pi.d_ccp, pi.d_crow, pi.d_cpos, nnz, a->L,
                                  a->NB, ly);
            else if (nc == 2)
                SPION_HYB_COL_LDS(ST, false, 2, Q, dO, nullptr, dS, P, dK, dV, pi.d_ccp, pi.d_crow, pi.d_cpos, nnz, a->L,
                                  a->NB, ly);
            if (nc) return;
        }
        hipLaunchKernelGGL((elem_bwd_col_kernel<D, ST>), grid, dim3(64 * ELEM_WAVES), 0, a->hdr.stream, Q, dO, P, dS,
                           dK, dV, pi.d_ccp, pi.d_crow, pi.d_cpos, a->L, a->NB, nnz, ly);
    }
}

// krow: Kt is K itself, row-major [NB][L][d], not the transposed copy of the reference's ABI.
void sparse_forward(void* h, const float* Q, const float* Kt, const float* V, const float* Mask, float* Attn,
                    float* Out, const int* Offsets, const int* Columns, int nnz, bool mask_entry, bool krow) {
    SparseAttn* a = as_sparse(h, "attn_forward");
    if (!a) return;
    if (a->has_mask != mask_entry || a->is_bf16) {
        set_error("attn_forward: handle was created by the %s init", a->is_bf16 ? "bf16" : a->has_mask ? "mask" : "no-mask");
        return;
    }
    if (!Q || !Kt || !V || !Attn || !Out || !Offsets || (nnz > 0 && !Columns) || (mask_entry && !Mask)) {
        set_error("attn_forward: null pointer argument");
        return;
    }
    if (!ensure_pattern(a, Offsets, Columns, nnz)) return;
    if (a->pat.tiled) {
        a->last_path = 1;
        if (a->d == 32) {
            if (krow) {
                if (a->has_mask) launch_tile_fwd<32, true, true>(a, Q, Kt, V, Mask, Attn, Out, Offsets, nnz);
                else launch_tile_fwd<32, false, true>(a, Q, Kt, V, nullptr, Attn, Out, Offsets, nnz);
            } else {
                if (a->has_mask) launch_tile_fwd<32, true, false>(a, Q, Kt, V, Mask, Attn, Out, Offsets, nnz);
                else launch_tile_fwd<32, false, false>(a, Q, Kt, V, nullptr, Attn, Out, Offsets, nnz);
            }
        } else {
            if (krow) {  // the d = 64 kernels read the transposed operand only: make it
                if (!ensure_ws(&a->ws_trans, (size_t)a->NB * a->L * a->d)) return;
                if (transpose_last2(Kt, a->ws_trans, a->NB, a->L, a->d, a->hdr.stream) != 0) return;
                Kt = a->ws_trans;
            }
            if (a->has_mask) launch_tile_fwd<64, true, false>(a, Q, Kt, V, Mask, Attn, Out, Offsets, nnz);
            else launch_tile_fwd<64, false, false>(a, Q, Kt, V, nullptr, Attn, Out, Offsets, nnz);
        }
        check_launch("tile_fwd_kernel");
        return;
    }
    a->last_path = 2;
    float* hyb_ocopy = a->pat.hybrid ? ocache_for_forward(a, Attn) : nullptr;
    if (!hyb_ocopy) ocache_drop(a, Attn);
    const float* Krm = Kt;  // the element kernels read K row-major
    if (!krow) {
        if (!ensure_ws(&a->ws_trans, (size_t)a->NB * a->L * a->d)) return;
        launch_transpose(a, Kt, a->ws_trans);
        Krm = a->ws_trans;
    }
    if (a->pat.hybrid) {
        launch_hyb_fwd<false>(a, Q, Krm, V, Mask, Attn, Out, hyb_ocopy, Offsets, nnz, Layouts{});
        return;
    }
    switch (a->d) {
        case 16: launch_elem_fwd<16>(a, Q, Krm, V, Mask, Attn, Out, Offsets, Columns, nnz); break;
        case 32: launch_elem_fwd<32>(a, Q, Krm, V, Mask, Attn, Out, Offsets, Columns, nnz); break;
        case 64: launch_elem_fwd<64>(a, Q, Krm, V, Mask, Attn, Out, Offsets, Columns, nnz); break;
        default: launch_elem_fwd<128>(a, Q, Krm, V, Mask, Attn, Out, Offsets, Columns, nnz); break;
    }
    check_launch("elem_fwd_kernel");
}

// Out (optional): the forward's output, for callers that still have it; the row sums g_i = dO_i . O_i then come
// from it and no kept copy is looked up.  vrow: Vt is V itself, row-major [NB][L][d].
void sparse_backward(void* h, const float* Q, const float* K, const float* Vt, const float* P, const float* dO,
                     float* dP, float* dS, float* dQ, float* dK, float* dV, const int* Offsets, const int* Columns,
                     int nnz, const float* Out, bool vrow) {
    SparseAttn* a = as_sparse(h, "attn_backward");
    if (!a) return;
    (void)dP;
    if (a->is_bf16) {
        set_error("attn_backward: handle was created by the bf16 init");
        return;
    }
    if (!Q || !K || !Vt || !P || !dO || !dQ || !dK || !dV || !Offsets || (nnz > 0 && !Columns)) {
        set_error("attn_backward: null pointer argument");
        return;
    }
    if (!ensure_pattern(a, Offsets, Columns, nnz)) return;
    if (a->pat.tiled) {
        a->last_path = 1;
        if (!ensure_ws(&a->ws_rowsum, (size_t)a->NB * a->L)) return;
        if (a->d == 32) {
            if (vrow) launch_tile_bwd<32, true>(a, Q, K, Vt, P, dO, dQ, dK, dV, Offsets, nnz, Out);
            else launch_tile_bwd<32, false>(a, Q, K, Vt, P, dO, dQ, dK, dV, Offsets, nnz, Out);
        } else {
            if (vrow) {
                if (!ensure_ws(&a->ws_trans, (size_t)a->NB * a->L * a->d)) return;
                if (transpose_last2(Vt, a->ws_trans, a->NB, a->L, a->d, a->hdr.stream) != 0) return;
                Vt = a->ws_trans;
            }
            launch_tile_bwd<64, false>(a, Q, K, Vt, P, dO, dQ, dK, dV, Offsets, nnz, Out);
        }
        check_launch("tile_bwd kernels");
        return;
    }
    a->last_path = 2;
    if (!dS) {
        set_error("attn_backward: the element path needs the dS scratch buffer");
        return;
    }
    const float* Vrm = Vt;  // the element kernels read V row-major
    if (!vrow) {
        if (!ensure_ws(&a->ws_trans, (size_t)a->NB * a->L * a->d)) return;
        launch_transpose(a, Vt, a->ws_trans);
        Vrm = a->ws_trans;
    }
    if (a->pat.hybrid) {
        // the hybrid kernels take the row sums from the forward's output (the caller's, or the handle's kept copy);
        // without it the gather kernels below serve the same P
        const float* o = Out ? Out : ocache_for_backward(a, P);
        if (o) {
            launch_hyb_bwd<false>(a, Q, K, Vrm, P, dO, o, dS, dQ, dK, dV, nnz, Layouts{});
            return;
        }
    }
    switch (a->d) {
        case 16: launch_elem_bwd<16>(a, Q, K, Vrm, P, dO, dS, dQ, dK, dV, Offsets, Columns, nnz); break;
        case 32: launch_elem_bwd<32>(a, Q, K, Vrm, P, dO, dS, dQ, dK, dV, Offsets, Columns, nnz); break;
        case 64: launch_elem_bwd<64>(a, Q, K, Vrm, P, dO, dS, dQ, dK, dV, Offsets, Columns, nnz); break;
        default: launch_elem_bwd<128>(a, Q, K, Vrm, P, dO, dS, dQ, dK, dV, Offsets, Columns, nnz); break;
    }
    check_launch("elem_bwd kernels");
}

// -------------------------------------------------------------------------------------------------
// Backward for callers that must not allocate (code under HIP graph capture, serving loops, harnesses that
// forbid hipMalloc): the row sums -g [NB][L] that the row pass leaves for the column pass go to a file-scope
// device array instead of the handle's workspace.  Every GPU holds its own copy of the array at its own
// address, looked up once per device with hipGetSymbolAddress; host code never uses the array's name as an
// address.  All calls on one GPU share the array: calls that overlap on one GPU race.
// -------------------------------------------------------------------------------------------------
constexpr size_t NOALLOC_MAX_ROWS = size_t(1) << 20;  // num_batches * seq_len; 4 MiB per GPU
static __device__ __align__(256) float scratch[NOALLOC_MAX_ROWS];
constexpr int NOALLOC_MAX_DEVICES = 64;
static float* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};
static std::mutex g_scratch_mutex;

// Address of `scratch` on the current device (nullptr and, if `report`, an error when it cannot be had).
static float* noalloc_scratch(bool report) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NOALLOC_MAX_DEVICES) {
        (void)hipGetLastError();
        if (report) set_error("spion_attn_backward_noalloc: no current device (or device index >= %d)", NOALLOC_MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            if (report) set_error("spion_attn_backward_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = static_cast<float*>(p);
    }
    return g_scratch_ptr[dev];
}

size_t sparse_noalloc_max_rows() { return NOALLOC_MAX_ROWS; }

void sparse_backward_noalloc(void* h, const float* Q, const float* K, const float* V, const float* P, const float* Out,
                             const float* dO, float* dQ, float* dK, float* dV, const int* Offsets, const int* Columns,
                             int nnz) {
    const char* who = "spion_attn_backward_noalloc";
    SparseAttn* a = as_sparse(h, who);
    if (!a) return;
    if (a->is_bf16) {
        set_error("%s: handle was created by the bf16 init", who);
        return;
    }
    if (!Q || !K || !V || !P || !Out || !dO || !dQ || !dK || !dV || !Offsets || (nnz > 0 && !Columns)) {
        set_error("%s: null pointer argument (Out is required)", who);
        return;
    }
    if ((size_t)a->NB * (size_t)a->L > NOALLOC_MAX_ROWS) {
        set_error("%s: num_batches * seq_len = %lld exceeds the %lld rows of the built-in scratch array", who,
                  (long long)a->NB * a->L, (long long)NOALLOC_MAX_ROWS);
        return;
    }
    if (a->d != 32) {
        set_error("%s: emb_dim %d unsupported (32 only: other sizes need workspace the library would have to allocate)",
                  who, a->d);
        return;
    }
    // the analysed pattern must be on file: analysing one allocates
    bool known = a->pat.valid && a->pat.key_off == Offsets && a->pat.key_col == Columns && a->pat.key_nnz == nnz;
    for (int i = 0; i < SparseAttn::PAT_SLOTS && !known; ++i) {
        const PatternIndex& pi = a->pats[i];
        if (pi.valid && pi.key_off == Offsets && pi.key_col == Columns && pi.key_nnz == nnz) {
            a->pat_stamp[i] = ++a->pat_clock;
            a->pat = pi;
            known = true;
        }
    }
    if (!known) {
        set_error("%s: this (Offsets, Columns, nnz) has not been analysed on this handle yet; run a forward or "
                  "spion_register_pattern first", who);
        return;
    }
    if (!a->pat.tiled) {
        set_error("%s: the pattern is not a union of aligned 32x32 tiles (the element kernels need a scratch of "
                  "num_batches * nnz floats from the caller: use spion_attn_backward_rowmajor)", who);
        return;
    }
    float* rowsum = noalloc_scratch(true);
    if (!rowsum) return;
    a->last_path = 1;
    launch_tile_bwd<32, true>(a, Q, K, V, P, dO, dQ, dK, dV, Offsets, nnz, Out, Layouts{}, rowsum);
    check_launch("tile_bwd kernels");
}

// Heads that are views of other memory (the [B][L][H*d] output of a projection seen as [B][H][L][d]): the tile
// kernels for d = 32 take the three strides of each tensor group and read / write the views in place.
static bool check_layout(const char* who, const char* what, const SparseAttn* a, int heads, const HeadLayout& y) {
    if (y.ld < a->d || y.ld % 4 || y.hstride % 4 || y.bstride % 4 || y.hstride < 0 || y.bstride < 0) {
        set_error("%s: %s layout: strides must be non-negative multiples of 4 floats and the row stride >= emb_dim", who,
                  what);
        return false;
    }
    // every byte offset inside one head's slice is a 32-bit quantity in the kernels
    if ((long long)a->L * y.ld >= (1ll << 29)) {
        set_error("%s: %s layout: seq_len * row stride = %lld floats exceeds 2^29", who, what, (long long)a->L * y.ld);
        return false;
    }
    (void)heads;
    return true;
}
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static SparseAttn* strided_handle(void* h, const char* who, const int* Offsets, const int* Columns, int nnz, int heads) {
    SparseAttn* a = as_sparse(h, who);
    if (!a) return nullptr;
    if (a->is_bf16) {
        set_error("%s: handle was created by the bf16 init", who);
        return nullptr;
    }
    if (heads <= 0 || a->NB % heads) {
        set_error("%s: heads = %d does not divide num_batches = %d", who, heads, a->NB);
        return nullptr;
    }
    if (!Offsets || (nnz > 0 && !Columns)) {
        set_error("%s: null pointer argument", who);
        return nullptr;
    }
    if (!ensure_pattern(a, Offsets, Columns, nnz)) return nullptr;
    if (a->pat.tiled && !tile_supported(a->d)) {  // cannot happen: tile patterns are only recognised for 32 and 64
        set_error("%s: emb_dim %d has no tile kernels", who, a->d);
        return nullptr;
    }
    return a;
}

void sparse_forward_strided(void* h, const float* Q, const float* K, const float* V, const float* Mask, float* Attn,
                            float* Out, const int* Offsets, const int* Columns, int nnz, int heads,
                            const HeadLayout& in, const HeadLayout& out) {
    const char* who = "attn_forward_strided";
    SparseAttn* a = strided_handle(h, who, Offsets, Columns, nnz, heads);
    if (!a) return;
    if (a->has_mask != (Mask != nullptr)) {
        set_error("%s: handle was created by the %s init", who, a->has_mask ? "mask" : "no-mask");
        return;
    }
    if (!Q || !K || !V || !Attn || !Out) {
        set_error("%s: null pointer argument", who);
        return;
    }
    if (!aligned16(Q) || !aligned16(K) || !aligned16(V) || !aligned16(Out)) {
        set_error("%s: operand pointers must be 16-byte aligned", who);
        return;
    }
    if (!check_layout(who, "input", a, heads, in) || !check_layout(who, "output", a, heads, out)) return;
    if (!layout_is_injective(out, a->NB / heads, heads, a->L, a->d)) {
        set_error("%s: the output layout maps two elements to one address", who);
        return;
    }
    Layouts ly{};
    ly.in = in;
    ly.out = out;
    ly.grad = out;
    ly.H = heads;
    if (!a->pat.tiled) {
        ocache_drop(a, Attn);  // the backward of these entry points is handed Out
        if (a->pat.hybrid) {
            launch_hyb_fwd<true>(a, Q, K, V, Mask, Attn, Out, nullptr, Offsets, nnz, ly);
            return;
        }
        a->last_path = 2;
        switch (a->d) {
            case 16: launch_elem_fwd<16, true>(a, Q, K, V, Mask, Attn, Out, Offsets, Columns, nnz, ly); break;
            case 32: launch_elem_fwd<32, true>(a, Q, K, V, Mask, Attn, Out, Offsets, Columns, nnz, ly); break;
            case 64: launch_elem_fwd<64, true>(a, Q, K, V, Mask, Attn, Out, Offsets, Columns, nnz, ly); break;
            default: launch_elem_fwd<128, true>(a, Q, K, V, Mask, Attn, Out, Offsets, Columns, nnz, ly); break;
        }
        check_launch("elem_fwd_kernel");
        return;
    }
    a->last_path = 1;
    if (a->d == 32) {
        if (a->has_mask) launch_tile_fwd<32, true, true, true>(a, Q, K, V, Mask, Attn, Out, Offsets, nnz, ly);
        else launch_tile_fwd<32, false, true, true>(a, Q, K, V, nullptr, Attn, Out, Offsets, nnz, ly);
    } else {
        if (a->has_mask) launch_tile_fwd<64, true, true, true>(a, Q, K, V, Mask, Attn, Out, Offsets, nnz, ly);
        else launch_tile_fwd<64, false, true, true>(a, Q, K, V, nullptr, Attn, Out, Offsets, nnz, ly);
    }
    check_launch("tile_fwd_kernel");
}

void sparse_backward_strided(void* h, const float* Q, const float* K, const float* V, const float* P, const float* Out,
                             const float* dO, float* dQ, float* dK, float* dV, const int* Offsets, const int* Columns,
                             int nnz, int heads, const HeadLayout& in, const HeadLayout& out, const HeadLayout& grad) {
    const char* who = "attn_backward_strided";
    SparseAttn* a = strided_handle(h, who, Offsets, Columns, nnz, heads);
    if (!a) return;
    if (!Q || !K || !V || !P || !Out || !dO || !dQ || !dK || !dV) {
        set_error("%s: null pointer argument", who);
        return;
    }
    if (!aligned16(Q) || !aligned16(K) || !aligned16(V) || !aligned16(Out) || !aligned16(dO) || !aligned16(dQ) ||
        !aligned16(dK) || !aligned16(dV)) {
        set_error("%s: operand pointers must be 16-byte aligned", who);
        return;
    }
    if (!check_layout(who, "input", a, heads, in) || !check_layout(who, "output", a, heads, out) ||
        !check_layout(who, "gradient", a, heads, grad))
        return;
    if (!layout_is_injective(grad, a->NB / heads, heads, a->L, a->d)) {
        set_error("%s: the gradient layout maps two elements to one address", who);
        return;
    }
    if (!ensure_ws(&a->ws_rowsum, (size_t)a->NB * a->L)) return;
    Layouts ly{};
    ly.in = in;
    ly.out = out;
    ly.grad = grad;
    ly.H = heads;
    if (!a->pat.tiled) {
        // these entry points have no dS argument: the scratch is the handle's (grown outside graph capture only)
        if (!ensure_ws_grow(a, &a->ws_ds, &a->ws_ds_count, (size_t)a->NB * (size_t)std::max(nnz, 1), who)) return;
        if (a->pat.hybrid) {
            launch_hyb_bwd<true>(a, Q, K, V, P, dO, Out, a->ws_ds, dQ, dK, dV, nnz, ly);
            return;
        }
        a->last_path = 2;
        switch (a->d) {
            case 16: launch_elem_bwd<16, true>(a, Q, K, V, P, dO, a->ws_ds, dQ, dK, dV, Offsets, Columns, nnz, ly); break;
            case 32: launch_elem_bwd<32, true>(a, Q, K, V, P, dO, a->ws_ds, dQ, dK, dV, Offsets, Columns, nnz, ly); break;
            case 64: launch_elem_bwd<64, true>(a, Q, K, V, P, dO, a->ws_ds, dQ, dK, dV, Offsets, Columns, nnz, ly); break;
            default: launch_elem_bwd<128, true>(a, Q, K, V, P, dO, a->ws_ds, dQ, dK, dV, Offsets, Columns, nnz, ly); break;
        }
        check_launch("elem_bwd kernels");
        return;
    }
    a->last_path = 1;
    if (a->d == 32) launch_tile_bwd<32, true, true>(a, Q, K, V, P, dO, dQ, dK, dV, Offsets, nnz, Out, ly);
    else launch_tile_bwd<64, true, true>(a, Q, K, V, P, dO, dQ, dK, dV, Offsets, nnz, Out, ly);
    check_launch("tile_bwd kernels");
}

// =================================================================================================
// bf16 family: row-major bf16 Q, K, V, dO, O and gradients; fp32 row statistics; tile patterns only
// =================================================================================================
void* sparse_bf16_init(int emb_dim, int seq_len, int num_batches, int block_size) {
    if (emb_dim != 32 && emb_dim != 64) {
        set_error("bf16 init: emb_dim %d unsupported (32 or 64)", emb_dim);
        return nullptr;
    }
    if (seq_len <= 0 || seq_len % 32) {
        set_error("bf16 init: seq_len %d must be a positive multiple of 32", seq_len);
        return nullptr;
    }
    SparseAttn* a = static_cast<SparseAttn*>(sparse_init(emb_dim, seq_len, num_batches, block_size, false));
    if (a) a->is_bf16 = true;
    return a;
}

static SparseAttn* as_bf16(void* h, const char* who, const int* Offsets, const int* Columns, int nnz) {
    SparseAttn* a = as_sparse(h, who);
    if (!a) return nullptr;
    if (!a->is_bf16) {
        set_error("%s: handle was not created by the bf16 init", who);
        return nullptr;
    }
    if (!ensure_pattern(a, Offsets, Columns, nnz)) return nullptr;
    if (!a->pat.tiled) {
        set_error("%s: the bf16 path needs a pattern made of aligned 32x32 tiles (block masks of block size 32, 64, ...)",
                  who);
        return nullptr;
    }
    return a;
}

// Workspace for the partial results of long strips: grows to the largest pattern seen (see ensure_ws_grow).
static bool ensure_part_ws(SparseAttn* a, int slots) {
    const size_t need = (size_t)a->NB * slots * (a->d == 32 ? bf16_slot_floats<32>() : bf16_slot_floats<64>());
    return ensure_ws_grow(a, &a->ws_part, &a->ws_part_floats, need, "bf16 attention");
}

// Bytes a tensor of [B][H][L][d] bf16 heads spans from its base pointer (the tile loads address whole tensors with
// 32-bit offsets); 0 if that is 4 GiB or more.
static unsigned bf16_extent(const SparseAttn* a, bool strided, const HeadLayout& y, int heads) {
    unsigned long long e;
    if (strided) {
        const int B = a->NB / heads;
        e = ((unsigned long long)(B - 1) * y.bstride + (unsigned long long)(heads - 1) * y.hstride +
             (unsigned long long)(a->L - 1) * y.ld + a->d) * 2ull;
    } else {
        e = (unsigned long long)a->NB * a->L * a->d * 2ull;
    }
    return e >= 0xfffffff0ull ? 0u : (unsigned)e;
}

template <bool ST>
static void bf16_forward_impl(SparseAttn* a, const void* Q, const void* K, const void* V, const float* Mask, void* Out,
                              float* Lse, const Layouts& ly) {
    PhaseRange phase("spion forward (bf16 kernels)");
    const PatternIndex& pi = a->pat;
    a->last_path = 1;
    const unsigned in_bytes = bf16_extent(a, ST, ly.in, ly.H), out_bytes = bf16_extent(a, ST, ly.out, ly.H);
    if (!in_bytes || !out_bytes) {
        set_error("bf16 attn_forward: the tensors span 4 GiB or more");
        return;
    }
    static const bool no_pairs = getenv("SPION_BF16_NO_PAIRS") != nullptr;
    const bool by_pairs = !ST && pi.plan_pair.lanes > 0 && !no_pairs;
    const Bf16Plan& plan = by_pairs ? pi.plan_pair : pi.plan_row;
    if (!ensure_part_ws(a, std::max(std::max(pi.plan_row.slots, pi.plan_col.slots), pi.plan_pair.slots))) return;
    const dim3 grid(plan.lanes), block(64), grid_m(plan.n_long * a->NB * (32 * a->d / 256));
    const __bf16 *q = static_cast<const __bf16*>(Q), *k = static_cast<const __bf16*>(K), *v = static_cast<const __bf16*>(V);
    __bf16* o = static_cast<__bf16*>(Out);
#define SPION_LAUNCH(DD, MM)                                                                                         \
    do {                                                                                                             \
        if (by_pairs)                                                                                                \
            hipLaunchKernelGGL((bf16_fwd_kernel<DD, MM, false, true>), grid, block, 0, a->hdr.stream, q, k, v, Mask, \
                               o, Lse, pi.d_tcol, plan.sched.items, plan.sched.lane_ptr, plan.sched.lane_ent, a->L, a->NB, a->scale, a->ws_part, plan.slots, ly,     \
                               in_bytes, out_bytes);                                                                            \
        else                                                                                                         \
            hipLaunchKernelGGL((bf16_fwd_kernel<DD, MM, ST, false>), grid, block, 0, a->hdr.stream, q, k, v, Mask,   \
                               o, Lse, pi.d_tcol, plan.sched.items, plan.sched.lane_ptr, plan.sched.lane_ent, a->L, a->NB, a->scale, a->ws_part, plan.slots, ly,     \
                               in_bytes, out_bytes);                                                                            \
        if (plan.n_long)                                                                                             \
            hipLaunchKernelGGL((bf16_merge_fwd_kernel<DD, ST>), grid_m, dim3(256), 0, a->hdr.stream, a->ws_part,     \
                               plan.d_longs, plan.n_long, plan.slots, o, Lse, a->L, ly.out, ly.H);                   \
    } while (0)
    if (a->d == 32) {
        if (Mask) SPION_LAUNCH(32, true);
        else SPION_LAUNCH(32, false);
    } else {
        if (Mask) SPION_LAUNCH(64, true);
        else SPION_LAUNCH(64, false);
    }
#undef SPION_LAUNCH
    check_launch("bf16_fwd_kernel");
}

template <bool ST>
static void bf16_backward_impl(SparseAttn* a, const void* Q, const void* K, const void* V, const float* Mask,
                               const void* Out, const float* Lse, const void* dO, void* dQ, void* dK, void* dV,
                               const Layouts& ly) {
    PhaseRange phase("spion backward (bf16 kernels)");
    const PatternIndex& pi = a->pat;
    a->last_path = 1;
    const unsigned in_bytes = bf16_extent(a, ST, ly.in, ly.H), out_bytes = bf16_extent(a, ST, ly.out, ly.H);
    const unsigned grad_bytes = bf16_extent(a, ST, ly.grad, ly.H);
    if (!in_bytes || !out_bytes || !grad_bytes) {
        set_error("bf16 attn_backward: the tensors span 4 GiB or more");
        return;
    }
    // {lse2, -g} of every strip, 64 floats per strip, from the row pass to the column pass
    if (!ensure_ws(&a->ws_rowsum, (size_t)a->NB * a->L * 2)) return;
    if (!ensure_part_ws(a, std::max(std::max(pi.plan_row.slots, pi.plan_col.slots), pi.plan_pair.slots))) return;
    // row pass: two strips per wavefront where the pattern has the pairs (SPION_BF16_ROW_PAIRS=0 keeps one strip)
    static const bool no_pairs = getenv("SPION_BF16_NO_PAIRS") != nullptr ||
                                 (getenv("SPION_BF16_ROW_PAIRS") && getenv("SPION_BF16_ROW_PAIRS")[0] == '0');
    const bool by_pairs = !ST && pi.plan_pair.lanes > 0 && !no_pairs;
    const Bf16Plan &pr = by_pairs ? pi.plan_pair : pi.plan_row, &pc = pi.plan_col;
    const dim3 grid_r(pr.lanes), grid_c(pc.lanes), block(64);
    const dim3 grid_mr(pr.n_long * a->NB * (32 * a->d / 256)), grid_mc(pc.n_long * a->NB * (2 * 32 * a->d / 256));
    const __bf16 *q = static_cast<const __bf16*>(Q), *k = static_cast<const __bf16*>(K), *v = static_cast<const __bf16*>(V);
    const __bf16 *o = static_cast<const __bf16*>(Out), *go = static_cast<const __bf16*>(dO);
    __bf16 *dq = static_cast<__bf16*>(dQ), *dk = static_cast<__bf16*>(dK), *dv = static_cast<__bf16*>(dV);
#define SPION_LAUNCH(DD, MM)                                                                                          \
    do {                                                                                                              \
        if (a->bwd_passes & 1) {                                                                                      \
            if (by_pairs)                                                                                             \
                hipLaunchKernelGGL((bf16_bwd_row_pair_kernel<DD, MM>), grid_r, block, 0, a->hdr.stream, q, k, v, go, \
                                   o, Lse, Mask, a->ws_rowsum, dq, pi.d_tcol, pr.sched.items, pr.sched.lane_ptr,      \
                                   pr.sched.lane_ent, a->L, a->NB, a->scale, a->ws_part, pr.slots, ly, in_bytes,      \
                                   out_bytes, grad_bytes);                                                            \
            else                                                                                                      \
            hipLaunchKernelGGL((bf16_bwd_row_kernel<DD, MM, ST>), grid_r, block, 0, a->hdr.stream, q, k, v, go, o,    \
                               Lse, Mask, a->ws_rowsum, dq, pi.d_tcol, pr.sched.items, pr.sched.lane_ptr, pr.sched.lane_ent, a->L, a->NB, a->scale, a->ws_part,   \
                               pr.slots, ly, in_bytes, out_bytes, grad_bytes);                                                               \
            if (pr.n_long)                                                                                            \
                hipLaunchKernelGGL((bf16_merge_sum_kernel<DD, ST>), grid_mr, dim3(256), 0, a->hdr.stream, a->ws_part, \
                                   pr.d_longs, pr.n_long, pr.slots, dq, (__bf16*)nullptr, a->L, ly.grad, ly.H);       \
        }                                                                                                             \
        if (a->bwd_passes & 2) {                                                                                      \
            hipLaunchKernelGGL((bf16_bwd_col_kernel<DD, MM, ST>), grid_c, block, 0, a->hdr.stream, q, k, v, go,       \
                               a->ws_rowsum, Mask, dk, dv, pi.d_tcdesc, pc.sched.items, pc.sched.lane_ptr, pc.sched.lane_ent, a->L, a->NB, a->scale, a->ws_part,  \
                               pc.slots, ly, in_bytes, out_bytes, grad_bytes);                                                    \
            if (pc.n_long)                                                                                            \
                hipLaunchKernelGGL((bf16_merge_sum_kernel<DD, ST>), grid_mc, dim3(256), 0, a->hdr.stream, a->ws_part, \
                                   pc.d_longs, pc.n_long, pc.slots, dk, dv, a->L, ly.grad, ly.H);                     \
        }                                                                                                             \
    } while (0)
    if (a->d == 32) {
        if (Mask) SPION_LAUNCH(32, true);
        else SPION_LAUNCH(32, false);
    } else {
        if (Mask) SPION_LAUNCH(64, true);
        else SPION_LAUNCH(64, false);
    }
#undef SPION_LAUNCH
    check_launch("bf16_bwd kernels");
}

void sparse_bf16_forward(void* h, const void* Q, const void* K, const void* V, const float* Mask, void* Out, float* Lse,
                         const int* Offsets, const int* Columns, int nnz) {
    if (!Q || !K || !V || !Out || !Lse || !Offsets || (nnz > 0 && !Columns)) {
        set_error("bf16 attn_forward: null pointer argument");
        return;
    }
    SparseAttn* a = as_bf16(h, "bf16 attn_forward", Offsets, Columns, nnz);
    if (!a) return;
    bf16_forward_impl<false>(a, Q, K, V, Mask, Out, Lse, Layouts{});
}

void sparse_bf16_backward(void* h, const void* Q, const void* K, const void* V, const float* Mask, const void* Out,
                          const float* Lse, const void* dO, void* dQ, void* dK, void* dV, const int* Offsets,
                          const int* Columns, int nnz) {
    if (!Q || !K || !V || !Out || !Lse || !dO || !dQ || !dK || !dV || !Offsets || (nnz > 0 && !Columns)) {
        set_error("bf16 attn_backward: null pointer argument");
        return;
    }
    SparseAttn* a = as_bf16(h, "bf16 attn_backward", Offsets, Columns, nnz);
    if (!a) return;
    bf16_backward_impl<false>(a, Q, K, V, Mask, Out, Lse, dO, dQ, dK, dV, Layouts{});
}

// The bf16 family on [B][H][L][d] views (strides in elements, multiples of 8; pointers 16-byte aligned).
static bool check_layout_bf16(const char* who, const char* what, const SparseAttn* a, const HeadLayout& y) {
    if (y.ld < a->d || y.ld % 8 || y.hstride % 8 || y.bstride % 8 || y.hstride < 0 || y.bstride < 0) {
        set_error("%s: %s layout: strides must be non-negative multiples of 8 elements and the row stride >= emb_dim",
                  who, what);
        return false;
    }
    if ((long long)a->L * y.ld >= (1ll << 29)) {
        set_error("%s: %s layout: seq_len * row stride = %lld elements exceeds 2^29", who, what, (long long)a->L * y.ld);
        return false;
    }
    return true;
}

void sparse_bf16_forward_strided(void* h, const void* Q, const void* K, const void* V, const float* Mask, void* Out,
                                 float* Lse, const int* Offsets, const int* Columns, int nnz, int heads,
                                 const HeadLayout& in, const HeadLayout& out) {
    const char* who = "bf16 attn_forward_strided";
    if (!Q || !K || !V || !Out || !Lse || !Offsets || (nnz > 0 && !Columns)) {
        set_error("%s: null pointer argument", who);
        return;
    }
    SparseAttn* a = as_bf16(h, who, Offsets, Columns, nnz);
    if (!a) return;
    if (heads <= 0 || a->NB % heads) {
        set_error("%s: heads = %d does not divide num_batches = %d", who, heads, a->NB);
        return;
    }
    if (!aligned16(Q) || !aligned16(K) || !aligned16(V) || !aligned16(Out)) {
        set_error("%s: operand pointers must be 16-byte aligned", who);
        return;
    }
    if (!check_layout_bf16(who, "input", a, in) || !check_layout_bf16(who, "output", a, out)) return;
    if (!layout_is_injective(out, a->NB / heads, heads, a->L, a->d)) {
        set_error("%s: the output layout maps two elements to one address", who);
        return;
    }
    Layouts ly{};
    ly.in = in;
    ly.out = out;
    ly.grad = out;
    ly.H = heads;
    bf16_forward_impl<true>(a, Q, K, V, Mask, Out, Lse, ly);
}

void sparse_bf16_backward_strided(void* h, const void* Q, const void* K, const void* V, const float* Mask,
                                  const void* Out, const float* Lse, const void* dO, void* dQ, void* dK, void* dV,
                                  const int* Offsets, const int* Columns, int nnz, int heads, const HeadLayout& in,
                                  const HeadLayout& out, const HeadLayout& grad) {
    const char* who = "bf16 attn_backward_strided";
    if (!Q || !K || !V || !Out || !Lse || !dO || !dQ || !dK || !dV || !Offsets || (nnz > 0 && !Columns)) {
        set_error("%s: null pointer argument", who);
        return;
    }
    SparseAttn* a = as_bf16(h, who, Offsets, Columns, nnz);
    if (!a) return;
    if (heads <= 0 || a->NB % heads) {
        set_error("%s: heads = %d does not divide num_batches = %d", who, heads, a->NB);
        return;
    }
    if (!aligned16(Q) || !aligned16(K) || !aligned16(V) || !aligned16(Out) || !aligned16(dO) || !aligned16(dQ) ||
        !aligned16(dK) || !aligned16(dV)) {
        set_error("%s: operand pointers must be 16-byte aligned", who);
        return;
    }
    if (!check_layout_bf16(who, "input", a, in) || !check_layout_bf16(who, "output", a, out) ||
        !check_layout_bf16(who, "gradient", a, grad))
        return;
    if (!layout_is_injective(grad, a->NB / heads, heads, a->L, a->d)) {
        set_error("%s: the gradient layout maps two elements to one address", who);
        return;
    }
    Layouts ly{};
    ly.in = in;
    ly.out = out;
    ly.grad = grad;
    ly.H = heads;
    bf16_backward_impl<true>(a, Q, K, V, Mask, Out, Lse, dO, dQ, dK, dV, ly);
}

// [batch][rows][cols] -> [batch][cols][rows], fp32.  Used by the host modules for the K^T / V^T operands
// the ABI asks for (models/attention_blockcuda.py:48,80 do it with permute + copy).
__global__ __launch_bounds__(256) void transpose_last2_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                              int rows, int cols) {
    __shared__ float tile[64][65];
    const size_t base = (size_t)blockIdx.z * rows * cols;
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
    for (int r = ty; r < 64; r += 4)
        if (r0 + r < rows && c0 + tx < cols) tile[r][tx] = in[base + (size_t)(r0 + r) * cols + c0 + tx];
    __syncthreads();
    for (int c = ty; c < 64; c += 4)
        if (c0 + c < cols && r0 + tx < rows) out[base + (size_t)(c0 + c) * rows + r0 + tx] = tile[tx][c];
}

// Same for narrow matrices (cols = 32 or 64, the head dimension) with rows a multiple of 256: a work-group
// moves 256 rows, reading 16 bytes per thread and writing 1 KB runs of each output row.
template <int COLS>
__global__ __launch_bounds__(256) void transpose_narrow_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                               int rows) {
    __shared__ float tile[256][COLS + 1];
    const size_t base = (size_t)blockIdx.y * rows * COLS;
    const int r0 = blockIdx.x * 256, t = threadIdx.x;
    const float4* src = reinterpret_cast<const float4*>(in + base + (size_t)r0 * COLS);
#pragma unroll
    for (int k = 0; k < COLS / 4; ++k) {
        const int e = t + 256 * k;  // float4 index inside the 256 x COLS slab
        const float4 v = src[e];
        const int r = e / (COLS / 4), c = (e % (COLS / 4)) * 4;
        tile[r][c] = v.x;
        tile[r][c + 1] = v.y;
        tile[r][c + 2] = v.z;
        tile[r][c + 3] = v.w;
    }
    __syncthreads();
#pragma unroll 8
    for (int c = 0; c < COLS; ++c) out[base + (size_t)c * rows + r0 + t] = tile[t][c];
}

int transpose_last2(const float* in, float* out, int batch, int rows, int cols, hipStream_t stream) {
    if (!in || !out || batch <= 0 || rows <= 0 || cols <= 0 || batch > 65535) {
        set_error("spion_transpose_last2: bad arguments");
        return 1;
    }
    if ((cols == 32 || cols == 64) && rows % 256 == 0) {
        const dim3 grid(rows / 256, batch);
        if (cols == 32) hipLaunchKernelGGL(transpose_narrow_kernel<32>, grid, dim3(256), 0, stream, in, out, rows);
        else hipLaunchKernelGGL(transpose_narrow_kernel<64>, grid, dim3(256), 0, stream, in, out, rows);
        return check_launch("transpose_narrow_kernel") ? 0 : 1;
    }
    dim3 grid((cols + 63) / 64, (rows + 63) / 64, batch);
    hipLaunchKernelGGL(transpose_last2_kernel, grid, dim3(256), 0, stream, in, out, rows, cols);
    return check_launch("transpose_last2_kernel") ? 0 : 1;
}

void sparse_invalidate(void* h) {
    SparseAttn* a = as_sparse(h, "spion_invalidate_pattern");
    if (a) a->release_patterns();
}
int sparse_last_path(void* h) {
    SparseAttn* a = as_sparse(h, "spion_last_path");
    return a ? a->last_path : 0;
}
// The schedule build_bf16_plan makes for a tile list, copied out for inspection (host only: nothing is launched or
// allocated on a device).  Returns the number of lanes; counts = {ints in items, ints in lane_ent, ints in longs,
// workspace slots}.  Arrays that are null or too small (cap_* in ints) are left alone.
int sparse_debug_bf16_plan(const int* ptr, int nstrips, int pairs, int NB, int lanes_wanted, int* items, int cap_items,
                           int* lane_ptr, int cap_ptr, int* lane_ent, int cap_ent, int* longs, int cap_longs,
                           int* counts) {
    if (!ptr || nstrips < 0 || NB <= 0 || lanes_wanted <= 0) return -1;
    const std::vector<int> p(ptr, ptr + nstrips + 1);
    const Bf16PlanHost plan = build_bf16_plan(p, nstrips, pairs != 0, NB, lanes_wanted);
    auto copy = [](const std::vector<int>& v, int* out, int cap) {
        if (out && (size_t)cap >= v.size()) std::copy(v.begin(), v.end(), out);
    };
    copy(plan.items, items, cap_items);
    copy(plan.lane_ptr, lane_ptr, cap_ptr);
    copy(plan.lane_ent, lane_ent, cap_ent);
    copy(plan.longs, longs, cap_longs);
    if (counts) {
        counts[0] = (int)plan.items.size();
        counts[1] = (int)plan.lane_ent.size();
        counts[2] = (int)plan.longs.size();
        counts[3] = plan.slots;
    }
    return plan.lanes;
}

int sparse_debug_counter(void* h, int which) {
    SparseAttn* a = as_sparse(h, "spion_debug_counter");
    if (!a) return -1;
    return which == 0 ? a->analyses_from_device : which == 1 ? a->analyses_from_host
         : which == 2 ? (int)a->retired.size() : -1;
}
void sparse_set_bwd_passes(void* h, int mask) {
    SparseAttn* a = as_sparse(h, "spion_set_backward_passes");
    if (a) a->bwd_passes = mask & 3;
}
void sparse_use_ocache(void* h, int on) {
    SparseAttn* a = as_sparse(h, "spion_use_output_cache");
    if (!a) return;
    a->use_ocache = on != 0;
    for (auto& sl : a->oslot) sl.key = nullptr;
}
void sparse_force_element(void* h, int on) {
    SparseAttn* a = as_sparse(h, "spion_force_element_path");
    if (!a) return;
    a->force_element = on != 0;
    a->release_patterns();
}

}  // namespace spion
