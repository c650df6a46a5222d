// Dense-phase attention (forward + backward) for gfx950: ordinary softmax attention that also
// materialises the full probability map, which the dense training phase hands to pattern discovery.
//
// Operand layouts are the reference's column-major ones (models/attn.cu:179-262,
// models/attention_cuda.py:18-74): Qt/Vt/dOt and all gradients are feature-major [NB][d][L], K (forward) and
// V (backward) are row-major [NB][L][d], and the map is stored key-major: Attn[h][j][i] = P[i][j].
// One work-group owns 32 queries (forward, row pass) or 32 keys (column pass) of one head and walks all
// L/32 tiles of the other dimension with v_mfma_f32_32x32x2_f32; see tile_ops.h for the register layout.
#include "common.h"
#include "tile_kernels.h"
#include "../../include/spion_hip.h"

#include <cmath>
#include <cstdlib>

namespace spion {

constexpr int DENSE_WAVES = 4;

template <int D, bool MASK>
__global__ __launch_bounds__(64 * DENSE_WAVES) void dense_fwd_kernel(
    const float* __restrict__ Qt, const float* __restrict__ K, const float* __restrict__ Vt,
    const float* __restrict__ pen, float* __restrict__ Attn, float* __restrict__ Out, float* __restrict__ OutCopy,
    int L, int nbr, int NB, float scale) {
    constexpr int WAVES = DENSE_WAVES;
    __shared__ float lds[WAVES * (D / 32) * 16 * 64];
    __shared__ float lds_m[WAVES][32], lds_z[WAVES][32];
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, I = item % nbr;
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const size_t hb = (size_t)bh * L * D;
    const float* penh = MASK ? pen + (size_t)bh * L : nullptr;
    float* Ah = Attn + (size_t)bh * L * L + I * 32 + li;

    float q[D / 2];
    load_cols<D>(Qt + hb, L, I * 32, li, h, q);

    float m = -10.f, z = 0.f;  // models/attn.cu:17
    for (int J = w; J < nbr; J += WAVES) {
        float k[D / 2];
        load_rows<D>(K + hb, J * 32, li, h, k);
        f32x16 s = mma_feat<D>(k, q);  // s[r] = q_i . k_j, i = I*32+li, j = J*32+acc_row(r,h)
        float v[16], tm = m;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            v[r] = s[r] * scale;
            if (MASK) v[r] -= penh[J * 32 + acc_row(r, h)];
            tm = fmaxf(tm, v[r]);
        }
        float zz = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) zz += __expf(v[r] - tm);
        z = z * __expf(m - tm) + zz;
        m = tm;
    }
    {
        float m2 = __shfl_xor(m, 32, 64), z2 = __shfl_xor(z, 32, 64);
        float M = fmaxf(m, m2);
        z = z * __expf(m - M) + z2 * __expf(m2 - M);
        m = M;
        if (h == 0) {
            lds_m[w][li] = m;
            lds_z[w][li] = z;
        }
        __syncthreads();
        float Mx = lds_m[0][li];
#pragma unroll
        for (int ww = 1; ww < WAVES; ++ww) Mx = fmaxf(Mx, lds_m[ww][li]);
        float Z = 0.f;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) Z += lds_z[ww][li] * __expf(lds_m[ww][li] - Mx);
        m = Mx;
        z = Z;
    }
    const float rinv = 1.0f / z;

    f32x16 o[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) o[c] = (f32x16){0};
    for (int J = w; J < nbr; J += WAVES) {
        float k[D / 2];
        load_rows<D>(K + hb, J * 32, li, h, k);
        f32x16 s = mma_feat<D>(k, q);
        float p[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float v = s[r] * scale;
            if (MASK) v -= penh[J * 32 + acc_row(r, h)];
            p[r] = __expf(v - m) * rinv;
            // the map is written once and is far larger than the caches: non-temporal
            __builtin_nontemporal_store(p[r], &Ah[(size_t)(J * 32 + acc_row(r, h)) * L]);
        }
        mma_tile_t<D>(p, Vt + hb, L, J * 32, li, h, o);
    }
    reduce_store<D, WAVES, true>(o, Out + hb, I * 32, w, li, h, lds, L);
    if (OutCopy) {  // kept by the handle for the backward's row sums
        __syncthreads();
        reduce_store<D, WAVES, true>(o, OutCopy + hb, I * 32, w, li, h, lds, L);
    }
}

// Forward for d = 32 and L <= 2048: the register-resident scheme of the sparse forward (tile_kernels.h) on the
// dense layouts.  Each of the WAVES wavefronts (four up to L = 1024, eight beyond) keeps the logit tiles of its
// share of the strip (at most MAXT) in registers, so a tile costs one QK^T chain and one PV chain instead of the
// two-sweep kernel's three; K and V tiles go from global memory straight into wave-private LDS tiles, map tiles
// change layout in a padded LDS tile and leave as four 16-byte instructions, non-temporally.
// RM: Q, V and Out are row-major head slices located by `ly` (heads possibly interleaved in [B][L][H*32] memory,
// tile_kernels.h) instead of the feature-major [NB][32][L] operands of the reference's ABI; K likewise.
// MEAN (row-major operands, eight wavefronts with at most four logit tiles each): the launch also accumulates the
// sum of the maps over the heads.  The grid is nbr x C work-groups instead of nbr x NB: work-group (c, I) walks the
// heads c, c + C, c + 2C, ... one after the other and adds every probability tile it writes to a register tile of
// its own, so the sum costs sixteen additions per tile and, once per work-group, the store of its [L][32] slab of
// Part[c] (key-major like the map).  The mean over batch and heads is then one small reduction of the C partial maps.
template <bool MASK, bool RM = false, int WAVES = 4, bool MEAN = false, int MAXT = 32 / WAVES>
SPION_TILE_KERNEL(WAVES) void dense_fwd_reg_kernel(
    const float* __restrict__ Qt, const float* __restrict__ K, const float* __restrict__ Vt,
    const float* __restrict__ pen, float* __restrict__ Attn, float* __restrict__ Out, float* __restrict__ OutCopy,
    int L, int nbr, int NB, float scale, Layouts ly, float* __restrict__ Part = nullptr, int C = 0) {
    static_assert(!MEAN || RM, "the mean-emitting forward takes row-major operands");
    constexpr int D = 32, KH = 16;
    __shared__ float lds[WAVES * 16 * 64];
    __shared__ float lds_m[WAVES][32], lds_z[WAVES][32];
    // per wavefront: one padded tile (the map tile on its way to memory), two 4 KB tiles filled straight from global
    // memory and the key penalties that travel with them
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][32 * TS + 2 * 1024 + (MASK ? 128 : 0)];
    const int item = xcd_remap(blockIdx.x, nbr * (MEAN ? C : NB));
    const int bh0 = item / nbr, I = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int nu = nbr > w ? (nbr - w + WAVES - 1) / WAVES : 0;  // key tiles w, w + WAVES, ... of this wavefront
    float* T = lds_t[w];  // map tile on its way to memory
    const char* Tb = reinterpret_cast<const char*>(T + 32 * TS);  // K tiles, later V tiles, alternately in two places
    const unsigned lb = lds_address(Tb);
    f32x16 total[MEAN ? MAXT : 1];
    if constexpr (MEAN) {
#pragma unroll
        for (int u = 0; u < MAXT; ++u) {
            total[u] = splat16(0.f);
        }
    }
    int bh = bh0;
    do {  // one head, or (MEAN) the heads bh0, bh0 + C, ...
    const size_t hb = (size_t)bh * L * D;
    size_t ib, ob, hbytes, obytes;
    int ild, old_;
    head_slice<RM, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<RM, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    const rsrc_t rQ = make_rsrc(Qt + ib, hbytes);
    const rsrc_t rA = make_rsrc(Attn + (size_t)bh * L * L, (size_t)L * L * 4);
    const u32x4 wK = rsrc_words(K + ib, hbytes), wV = rsrc_words(Vt + ib, hbytes);
    const u32x4 wM = rsrc_words(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
    const int alin = lin_voff(l, L);
    const int vld = RM ? ild : L, VSTEP = RM ? 32 * ild * 4 : 128;
    const int kl = DmaTileF32::voff(l, ild), kx = DmaTileF32::extra_step(ild);
    const int vl = DmaTileF32::voff(l, vld), vx = DmaTileF32::extra_step(vld);
    const float c2 = scale * LOG2E;

    float q[KH];
    if constexpr (RM) ldr_rows<D>(rQ, (li * ild + h * KH) * 4, I * 32 * ild * 4, q);
    else ldr_cols<D>(rQ, L, (h * KH * L + li) * 4, I * 128, q);
#pragma unroll
    for (int s = 0; s < KH; ++s) q[s] *= c2;

    float m = -10.f * LOG2E, z = 0.f;  // models/attn.cu:17
    f32x16 S[MAXT];
    {
        // K tile u + 1 (and its key penalties) is requested before the chain of tile u starts; loads into LDS and
        // the map's stores share one in-order counter (wait_vm)
        const auto a_k = DmaTileF32::own_addr(Tb, li, 4 * h, 1);  // K[key li][feature 16h + s]
        const char* Tm = Tb + 2 * DmaTileF32::TILE + 16 * h;
        constexpr int KOPS = MASK ? 5 : 4;
        auto issue_k = [&](int u) {
            const int J = w + u * WAVES;
            DmaTileF32::load(wK, lb + (u & 1) * DmaTileF32::TILE, kl, J * 32 * ild * 4, kx);
            if constexpr (MASK) dma_b32(wM, lb + 2 * DmaTileF32::TILE + (u & 1) * 256, l * 4, J * 128);
        };
        if (nu > 0) issue_k(0);
#pragma unroll
        for (int u = 0; u < MAXT; ++u) {
            if (u < nu) {
                if (u + 1 < MAXT && u + 1 < nu) {
                    issue_k(u + 1);
                    wait_vm<KOPS>();
                } else {
                    wait_vm<0>();
                }
                float kf[KH];
                DmaTileF32::get(a_k, kf, (u & 1) * DmaTileF32::TILE);
                f32x16 init = splat16(0.f);
                if constexpr (MASK) {  // minus the key penalties of the tile, log2 domain
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 x = *reinterpret_cast<const f32x4*>(Tm + (u & 1) * 256 + 32 * g);
                        init[4 * g + 0] = -LOG2E * x.x;
                        init[4 * g + 1] = -LOG2E * x.y;
                        init[4 * g + 2] = -LOG2E * x.z;
                        init[4 * g + 3] = -LOG2E * x.w;
                    }
                }
                wait_lgkm0();  // the tile's space is requested again one iteration on
                __builtin_amdgcn_sched_barrier(0);
                S[u] = mma_feat_init<D>(kf, q, init);  // S^T: register = key, lane = query
                m = max16(S[u], m);
            }
        }
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
    {
        if (h == 0) {
            lds_m[w][li] = m;
            lds_z[w][li] = z;
        }
        __syncthreads();
        float Mx = lds_m[0][li];
#pragma unroll
        for (int ww = 1; ww < WAVES; ++ww) Mx = fmaxf(Mx, lds_m[ww][li]);
        float Z = 0.f;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) Z += lds_z[ww][li] * __builtin_amdgcn_exp2f(lds_m[ww][li] - Mx);
        m = Mx;
        z = Z;
    }
    const float rinv = __builtin_amdgcn_exp2f(m_own - m) * (1.0f / z);

    f32x16 o[1] = {splat16(0.f)};  // O^T: register = feature, lane = query
    {
        // V tiles the same way, two ahead: request u + 2 goes out when tile u has been read.  What was issued after
        // the loads of tile u when its turn comes: the loads of tile u + 1 (if any) and the map stores of the one or
        // two tiles before it.
        const auto a_v = [&] {
            if constexpr (RM) return DmaTileF32::cols_addr(Tb, li, h);  // vb[s] = V[key acc_row(s, h)][feature li]
            else return DmaTileF32::own_addr(Tb, li, h, 2);
        }();
        auto issue_v = [&](int u) {
            DmaTileF32::load(wV, lb + (u & 1) * DmaTileF32::TILE, vl, (w + u * WAVES) * VSTEP, vx);
        };
        if (nu > 0) issue_v(0);
        if (MAXT > 1 && nu > 1) issue_v(1);
#pragma unroll
        for (int u = 0; u < MAXT; ++u) {
            if (u < nu) {
                const int J = w + u * WAVES;
                const int stores = u == 0 ? 0 : u == 1 ? 4 : 8;  // map stores issued after V tile u was requested
                wait_vm_upto(stores + (u + 1 < MAXT && u + 1 < nu ? 4 : 0));
                float p[16], vb[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) p[r] = S[u][r] * rinv;
                if constexpr (MEAN) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) total[u][r] += p[r];
                }
                lds_put_cols(T, li, h, p);  // T[key][query]: the map is stored key-major
                DmaTileF32::get(a_v, vb, (u & 1) * DmaTileF32::TILE);
                f32x4 pl[4];
                lds_get_lin(T, l, pl);
                wait_lgkm0();
                if (u + 2 < MAXT && u + 2 < nu) issue_v(u + 2);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < 16; ++s) o[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb[s], p[s], o[0], 0, 0, 0);
                str_tile_lin(rA, alin, (J * 32 * L + I * 32) * 4, L, pl);
            }
        }
    }
    if constexpr (RM) {
        reduce_store_rows<WAVES>(o[0], Out + ob, I * 32, w, li, h, lds, old_);
    } else {
        reduce_store<D, WAVES, true>(o, Out + hb, I * 32, w, li, h, lds, L);
        if (OutCopy) {
            __syncthreads();
            reduce_store<D, WAVES, true>(o, OutCopy + hb, I * 32, w, li, h, lds, L);
        }
    }
    if constexpr (MEAN) __syncthreads();  // the shared arrays are free for the next head
    bh += MEAN ? C : NB;
    } while (MEAN && bh < NB);
    if constexpr (MEAN) {
        const rsrc_t rS = make_rsrc(Part + (size_t)bh0 * L * L, (size_t)L * L * 4);
        const int alin = lin_voff(l, L);
#pragma unroll
        for (int u = 0; u < MAXT; ++u) {
            if (u < nu) {
                float p[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) p[r] = total[u][r];
                lds_put_cols(T, li, h, p);
                f32x4 pl[4];
                lds_get_lin(T, l, pl);
                str_tile_lin_cached(rS, alin, ((w + u * WAVES) * 32 * L + I * 32) * 4, L, pl);
            }
        }
    }
}

// Forward for d = 64, row-major operands, L <= 256 * WAVES: the same register-resident scheme.  A K or V tile is two 4 KB
// tiles (features 0..31 and 32..63) in one place per wavefront: the operands of tile u are read out into registers,
// then the space is requested for tile u + 1, whose loads have the chains of tile u (32 MFMA) to arrive.
template <bool MASK, int WAVES = 4>
SPION_TILE_KERNEL(WAVES) void dense_fwd_reg64_kernel(
    const float* __restrict__ Q, const float* __restrict__ K, const float* __restrict__ V,
    const float* __restrict__ pen, float* __restrict__ Attn, float* __restrict__ Out,
    int L, int nbr, int NB, float scale, Layouts ly) {
    constexpr int D = 64, KH = 32, MAXT = 8;
    __shared__ float lds[WAVES * 16 * 64];
    __shared__ float lds_m[WAVES][32], lds_z[WAVES][32];
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][32 * TS + 2 * 1024 + (MASK ? 64 : 0)];
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, I = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int nu = nbr > w ? (nbr - w + WAVES - 1) / WAVES : 0;  // key tiles w, w + WAVES, ... of this wavefront
    float* T = lds_t[w];  // map tile on its way to memory
    const char* Tb = reinterpret_cast<const char*>(T + 32 * TS);  // the two halves of a K tile, later of a V tile
    const unsigned lb = lds_address(Tb);
    size_t ib, ob, hbytes, obytes;
    int ild, old_;
    head_slice<true, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<true, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    const rsrc_t rA = make_rsrc(Attn + (size_t)bh * L * L, (size_t)L * L * 4);
    const u32x4 wK = rsrc_words(K + ib, hbytes), wV = rsrc_words(V + ib, hbytes);
    const u32x4 wM = rsrc_words(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
    const int alin = lin_voff(l, L);
    const int kl = DmaTileF32::voff(l, ild), kx = DmaTileF32::extra_step(ild);
    const float c2 = scale * LOG2E;
    auto issue = [&](const u32x4& r, int J) {
        DmaTileF32::load(r, lb, kl, J * 32 * ild * 4, kx);
        DmaTileF32::load(r, lb + DmaTileF32::TILE, kl, J * 32 * ild * 4 + 128, kx);
    };

    float q[KH];
    ldr_rows<D>(make_rsrc(Q + ib, hbytes), (li * ild + h * KH) * 4, I * 32 * ild * 4, q);
#pragma unroll
    for (int s = 0; s < KH; ++s) q[s] *= c2;
    settle(q);

    float m = -10.f * LOG2E, z = 0.f;  // models/attn.cu:17
    f32x16 S[MAXT];
    {
        const auto a_k = DmaTileF32::own8_addr(Tb + h * DmaTileF32::TILE, li);  // K[key li][feature 32h + s]
        const char* Tm = Tb + 2 * DmaTileF32::TILE + 16 * h;
        auto issue_k = [&](int u) {
            const int J = w + u * WAVES;
            issue(wK, J);
            if constexpr (MASK) dma_b32(wM, lb + 2 * DmaTileF32::TILE, l * 4, J * 128);
        };
        if (nu > 0) issue_k(0);
#pragma unroll
        for (int u = 0; u < MAXT; ++u) {
            if (u < nu) {
                wait_vm<0>();
                float kf[KH];
                DmaTileF32::get32(a_k, kf);
                f32x16 init = splat16(0.f);
                if constexpr (MASK) {  // minus the key penalties of the tile, log2 domain
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 x = *reinterpret_cast<const f32x4*>(Tm + 32 * g);
                        init[4 * g + 0] = -LOG2E * x.x;
                        init[4 * g + 1] = -LOG2E * x.y;
                        init[4 * g + 2] = -LOG2E * x.z;
                        init[4 * g + 3] = -LOG2E * x.w;
                    }
                }
                wait_lgkm0();
                if (u + 1 < MAXT && u + 1 < nu) issue_k(u + 1);
                __builtin_amdgcn_sched_barrier(0);
                S[u] = mma_feat_init<D>(kf, q, init);  // S^T: register = key, lane = query
                m = max16(S[u], m);
            }
        }
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
    if (h == 0) {
        lds_m[w][li] = m;
        lds_z[w][li] = z;
    }
    __syncthreads();
    {
        float Mx = lds_m[0][li];
#pragma unroll
        for (int ww = 1; ww < WAVES; ++ww) Mx = fmaxf(Mx, lds_m[ww][li]);
        float Z = 0.f;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) Z += lds_z[ww][li] * __builtin_amdgcn_exp2f(lds_m[ww][li] - Mx);
        m = Mx;
        z = Z;
    }
    const float rinv = __builtin_amdgcn_exp2f(m_own - m) * (1.0f / z);

    f32x16 o[2] = {splat16(0.f), splat16(0.f)};  // O^T: register = feature (+32), lane = query
    {
        const auto a_v = DmaTileF32::cols_addr(Tb, li, h);  // vb[c][s] = V[key acc_row(s, h)][feature 32c + li]
        if (nu > 0) issue(wV, w);
#pragma unroll
        for (int u = 0; u < MAXT; ++u) {
            if (u < nu) {
                const int J = w + u * WAVES;
                // in flight after the loads of V tile u: the four map stores of tile u - 1
                if (u == 0) wait_vm<0>();
                else wait_vm<4>();
                float p[16], vb[2][16];
#pragma unroll
                for (int r = 0; r < 16; ++r) p[r] = S[u][r] * rinv;
                lds_put_cols(T, li, h, p);  // T[key][query]: the map is stored key-major
                DmaTileF32::get(a_v, vb[0]);
                DmaTileF32::get(a_v, vb[1], DmaTileF32::TILE);
                f32x4 pl[4];
                lds_get_lin(T, l, pl);
                wait_lgkm0();
                if (u + 1 < MAXT && u + 1 < nu) issue(wV, w + (u + 1) * WAVES);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int c = 0; c < 2; ++c)
#pragma unroll
                    for (int s = 0; s < 16; ++s)
                        o[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb[c][s], p[s], o[c], 0, 0, 0);
                str_tile_lin(rA, alin, (J * 32 * L + I * 32) * 4, L, pl);
            }
        }
    }
    reduce_store_rows<WAVES>(o[0], Out + ob, I * 32, w, li, h, lds, old_);
    __syncthreads();
    reduce_store_rows<WAVES>(o[1], Out + ob + 32, I * 32, w, li, h, lds, old_);
}

// Forward for d = 32 and any L: two sweeps over the key tiles of a query strip, four wavefronts sharing the strip.
// Sweep 1 keeps a running maximum and sum of exponentials per wavefront (merged over the work-group afterwards);
// sweep 2 recomputes the logits with -M folded into the chain's initial accumulator, writes the map and
// accumulates O^T.  Tiles are fetched linearly one tile ahead and re-laid out in wave-private LDS tiles, as in
// the kernels above.  48 MFMA per tile against the 32 of the register-resident kernel, which is why that one is
// used whenever a strip's logits fit in the registers of four wavefronts.
// MEAN (row-major operands only): the launch also accumulates the sum of the maps over the heads.  The grid is
// nbr x C work-groups instead of nbr x NB: work-group (c, I) walks the heads c, c + C, c + 2C, ... one after the
// other and adds every map tile it writes to its own [L][32] slab of Part[c] (key-major like the map; plain
// read-modify-write, nobody else touches the slab), so the mean over batch and heads is one small reduction of the
// C partial maps afterwards instead of a second pass over all NB maps.
template <bool MASK, bool RM = false, bool MEAN = false>
SPION_TILE_KERNEL(4) void dense_fwd_sweep32_kernel(
    const float* __restrict__ Qt, const float* __restrict__ K, const float* __restrict__ Vt,
    const float* __restrict__ pen, float* __restrict__ Attn, float* __restrict__ Out, float* __restrict__ OutCopy,
    int L, int nbr, int NB, float scale, Layouts ly, float* __restrict__ Part = nullptr, int C = 0) {
    static_assert(!MEAN || RM, "the mean-emitting forward takes row-major operands");
    constexpr int D = 32, KH = 16, WAVES = 4;
    __shared__ float lds[WAVES * 16 * 64];
    __shared__ float lds_m[WAVES][32], lds_z[WAVES][32];
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][3 * 32 * TS];
    const int item = xcd_remap(blockIdx.x, nbr * (MEAN ? C : NB));
    const int bh0 = item / nbr, I = item % nbr;
    const int bh_step = MEAN ? C : NB;
    int bh = bh0;
    do {  // one head, or (MEAN) the heads bh0, bh0 + C, ...
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int nu = nbr > w ? (nbr - w + WAVES - 1) / WAVES : 0;
    const size_t hb = (size_t)bh * L * D;
    size_t ib, ob, hbytes, obytes;
    int ild, old_;
    head_slice<RM, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<RM, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    const rsrc_t rQ = make_rsrc(Qt + ib, hbytes), rK = make_rsrc(K + ib, hbytes), rV = make_rsrc(Vt + ib, hbytes);
    const rsrc_t rA = make_rsrc(Attn + (size_t)bh * L * L, (size_t)L * L * 4);
    const rsrc_t rS = make_rsrc(MEAN ? Part + (size_t)bh0 * L * L : Part, MEAN ? (size_t)L * L * 4 : 0);
    const rsrc_t rM = make_rsrc(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
    float* T = lds_t[w];          // map tile on its way to memory
    float* Tk = T + 32 * TS;
    float* Tv = T + 64 * TS;
    const int klin = lin_voff(l, ild), alin = lin_voff(l, L);
    const int vld = RM ? ild : L, vlin = lin_voff(l, vld), VSTEP = RM ? 32 * ild * 4 : 128;
    const float c2 = scale * LOG2E;

    float q[KH];
    if constexpr (RM) ldr_rows<D>(rQ, (li * ild + h * KH) * 4, I * 32 * ild * 4, q);
    else ldr_cols<D>(rQ, L, (h * KH * L + li) * 4, I * 128, q);
#pragma unroll
    for (int s = 0; s < KH; ++s) q[s] *= c2;

    struct Pre1 {
        f32x4 k[4];
        float pj[MASK ? 16 : 1];
    };
    struct Pre2 {
        f32x4 k[4], v[4];
        float pj[MASK ? 16 : 1];
    };
    auto penalties = [&](float (&pj)[MASK ? 16 : 1], int J) {
        if constexpr (MASK) {
            float t[16];
            ldr_4x4(rM, 16 * h, J * 128, t);
#pragma unroll
            for (int r = 0; r < 16; ++r) pj[r] = t[r];
        }
    };

    // ---- sweep 1: running maximum and sum over this wavefront's tiles (log2 domain) ----------------
    float m = -10.f * LOG2E, z = 0.f;  // models/attn.cu:17
    {
        Pre1 xa, xb;
        tile_pipeline(
            nu, xa, xb,
            [&](Pre1& x, int i) {
                const int J = w + min(i, nu - 1) * WAVES;
                ldr_tile_lin(rK, klin, J * 32 * ild * 4, ild, x.k);
                penalties(x.pj, J);
            },
            [&](Pre1& c, int) {
                lds_put_lin(Tk, l, c.k);
                float kf[KH];
                lds_get_feat32(Tk, li, h, kf);
                __builtin_amdgcn_sched_barrier(0);
                f32x16 init = splat16(0.f);
                if constexpr (MASK) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) init[r] = -LOG2E * c.pj[r];
                }
                const f32x16 S = mma_feat_init<D>(kf, q, init);  // register = key, lane = query
                const float mn = max16(S, m);
                z *= __builtin_amdgcn_exp2f(m - mn);
                m = mn;
#pragma unroll
                for (int r = 0; r < 16; ++r) z += __builtin_amdgcn_exp2f(S[r] - m);
            });
    }
    {   // the two half-waves, then the four wavefronts
        const float mo = __shfl_xor(m, 32, 64), zo = __shfl_xor(z, 32, 64);
        const float mn = fmaxf(m, mo);
        z = z * __builtin_amdgcn_exp2f(m - mn) + zo * __builtin_amdgcn_exp2f(mo - mn);
        m = mn;
        if (h == 0) {
            lds_m[w][li] = m;
            lds_z[w][li] = z;
        }
        __syncthreads();
        float Mx = lds_m[0][li];
#pragma unroll
        for (int ww = 1; ww < WAVES; ++ww) Mx = fmaxf(Mx, lds_m[ww][li]);
        float Z = 0.f;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) Z += lds_z[ww][li] * __builtin_amdgcn_exp2f(lds_m[ww][li] - Mx);
        m = Mx;
        z = Z;
    }
    const float rinv = 1.0f / z;
    const f32x16 minus_m = splat16(-m);

    // ---- sweep 2: probabilities, map tiles and O^T --------------------------------------------------
    f32x16 o[1] = {splat16(0.f)};  // O^T: register = feature, lane = query
    {
        Pre2 xa, xb;
        tile_pipeline(
            nu, xa, xb,
            [&](Pre2& x, int i) {
                const int J = w + min(i, nu - 1) * WAVES;
                ldr_tile_lin(rK, klin, J * 32 * ild * 4, ild, x.k);
                ldr_tile_lin(rV, vlin, J * VSTEP, vld, x.v);
                penalties(x.pj, J);
            },
            [&](Pre2& c, int i) {
                const int J = w + i * WAVES;
                f32x4 sum4[4];
                if constexpr (MEAN) {
                    if (bh != bh0) ldr_tile_lin_l2(rS, alin, (J * 32 * L + I * 32) * 4, L, sum4);
                }
                lds_put_lin(Tk, l, c.k);
                lds_put_lin(Tv, l, c.v);
                float kf[KH], vb[16];
                lds_get_feat32(Tk, li, h, kf);
                if constexpr (RM) lds_get_cols(Tv, li, h, vb);  // V[key acc_row(s, h)][feature li]
                else lds_get_rows(Tv, li, h, vb);
                __builtin_amdgcn_sched_barrier(0);
                f32x16 init = minus_m;
                if constexpr (MASK) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) init[r] -= LOG2E * c.pj[r];
                }
                const f32x16 S = mma_feat_init<D>(kf, q, init);  // logits minus the row maximum
                float p[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) p[r] = __builtin_amdgcn_exp2f(S[r]) * rinv;
                lds_put_cols(T, li, h, p);  // T[key][query]: the map is stored key-major
                f32x4 pl[4];
                lds_get_lin(T, l, pl);
#pragma unroll
                for (int s = 0; s < 16; ++s) o[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb[s], p[s], o[0], 0, 0, 0);
                str_tile_lin(rA, alin, (J * 32 * L + I * 32) * 4, L, pl);
                if constexpr (MEAN) {
                    if (bh != bh0) {
#pragma unroll
                        for (int k = 0; k < 4; ++k) pl[k] += sum4[k];
                    }
                    str_tile_lin_cached(rS, alin, (J * 32 * L + I * 32) * 4, L, pl);
                }
            });
    }
    if constexpr (RM) {
        reduce_store_rows<WAVES>(o[0], Out + ob, I * 32, w, li, h, lds, old_);
    } else {
        reduce_store<D, WAVES, true>(o, Out + hb, I * 32, w, li, h, lds, L);
        if (OutCopy) {
            __syncthreads();
            reduce_store<D, WAVES, true>(o, OutCopy + hb, I * 32, w, li, h, lds, L);
        }
    }
    if constexpr (MEAN) {
        // this wavefront's slab stores are complete before its loads of the next head; the barrier also frees the
        // shared arrays for the next head
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    bh += bh_step;
    } while (MEAN && bh < NB);
}

// Row pass: g_i = sum_j dP_ij P_ij (kept in G), dS = (dP*P - P*g)*scale, dQ^T = K^T-tiles . dS^T.
// HAVE_O: the handle kept Out of the forward that filled this map, so g_i = dO_i . O_i needs no sweep.
template <int D, bool HAVE_O>
__global__ __launch_bounds__(64 * DENSE_WAVES) void dense_bwd_row_kernel(
    const float* __restrict__ Kt, const float* __restrict__ V, const float* __restrict__ Attn,
    const float* __restrict__ dOt, const float* __restrict__ OutCopy, float* __restrict__ G,
    float* __restrict__ dQ, int L, int nbr, int NB, float scale) {
    constexpr int WAVES = DENSE_WAVES;
    __shared__ float lds[WAVES * (D / 32) * 16 * 64];
    __shared__ float lds_g[WAVES][32];
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, I = item % nbr;
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const size_t hb = (size_t)bh * L * D;
    const float* Ah = Attn + (size_t)bh * L * L + I * 32 + li;

    float go[D / 2];
    load_cols<D>(dOt + hb, L, I * 32, li, h, go);

    float g = 0.f;
    if (HAVE_O) {
        float oo[D / 2];
        load_cols<D>(OutCopy + hb, L, I * 32, li, h, oo);
#pragma unroll
        for (int s = 0; s < D / 2; ++s) g = fmaf(go[s], oo[s], g);
        g += __shfl_xor(g, 32, 64);
    } else {
        for (int J = w; J < nbr; J += WAVES) {
            float v[D / 2];
            load_rows<D>(V + hb, J * 32, li, h, v);
            f32x16 dp = mma_feat<D>(v, go);
#pragma unroll
            for (int r = 0; r < 16; ++r) g = fmaf(dp[r], Ah[(size_t)(J * 32 + acc_row(r, h)) * L], g);
        }
        g += __shfl_xor(g, 32, 64);
        if (h == 0) lds_g[w][li] = g;
        __syncthreads();
        g = 0.f;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) g += lds_g[ww][li];
    }
    if (w == 0 && h == 0) G[(size_t)bh * L + I * 32 + li] = -g;  // the column passes start their chains from it

    f32x16 acc[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) acc[c] = (f32x16){0};
    for (int J = w; J < nbr; J += WAVES) {
        float v[D / 2];
        load_rows<D>(V + hb, J * 32, li, h, v);
        f32x16 dp = mma_feat<D>(v, go);
        float ds[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float p = HAVE_O ? __builtin_nontemporal_load(&Ah[(size_t)(J * 32 + acc_row(r, h)) * L])
                                   : Ah[(size_t)(J * 32 + acc_row(r, h)) * L];
            ds[r] = (dp[r] * p - p * g) * scale;
        }
        mma_tile_t<D>(ds, Kt + hb, L, J * 32, li, h, acc);
    }
    reduce_store<D, WAVES, true>(acc, dQ + hb, I * 32, w, li, h, lds, L);
}

// Column pass: dK^T = Q^T-tiles . dS, dV^T = dO^T-tiles . P for 32 keys of one head.
template <int D>
__global__ __launch_bounds__(64 * DENSE_WAVES) void dense_bwd_col_kernel(
    const float* __restrict__ Qt, const float* __restrict__ V, const float* __restrict__ Attn,
    const float* __restrict__ dOt, const float* __restrict__ G, float* __restrict__ dK, float* __restrict__ dV,
    int L, int nbr, int NB, float scale) {
    constexpr int WAVES = DENSE_WAVES;
    __shared__ float lds[WAVES * (D / 32) * 16 * 64];
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, J = item % nbr;
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const size_t hb = (size_t)bh * L * D;
    const float* Arow = Attn + (size_t)bh * L * L + (size_t)(J * 32 + li) * L + 4 * h;
    const float* Gh = G + (size_t)bh * L;

    float v[D / 2];
    load_rows<D>(V + hb, J * 32, li, h, v);

    f32x16 ak[D / 32], av[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        ak[c] = (f32x16){0};
        av[c] = (f32x16){0};
    }
    for (int I = w; I < nbr; I += WAVES) {
        float go[D / 2];
        load_cols<D>(dOt + hb, L, I * 32, li, h, go);
        f32x16 dp = mma_feat<D>(go, v);  // dp[r] = dO_i . v_j, i = I*32+acc_row(r,h), j = J*32+li
        float p[16], ds[16];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            float4 pv = *reinterpret_cast<const float4*>(Arow + I * 32 + 8 * g4);
            p[4 * g4] = pv.x;
            p[4 * g4 + 1] = pv.y;
            p[4 * g4 + 2] = pv.z;
            p[4 * g4 + 3] = pv.w;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float g = -Gh[I * 32 + acc_row(r, h)];
            ds[r] = (dp[r] * p[r] - p[r] * g) * scale;
        }
        mma_tile_t<D>(ds, Qt + hb, L, I * 32, li, h, ak);
        mma_tile_t<D>(p, dOt + hb, L, I * 32, li, h, av);
    }
    reduce_store<D, WAVES, true>(ak, dK + hb, J * 32, w, li, h, lds, L);
    __syncthreads();
    reduce_store<D, WAVES, true>(av, dV + hb, J * 32, w, li, h, lds, L);
}

// Backward passes for d = 32 with the kept copy of Out: the schedule of the sparse tile kernels (tile_kernels.h)
// on the dense layouts.  Every operand tile -- V, K^T, Q^T, dO^T and the key-major map tile -- goes from global
// memory straight into a wave-private LDS tile, one tile ahead, and is read from there as MFMA operands; -g enters as
// the initial accumulator of the dP chain; the 1/sqrt(d) is applied to the 32 x d results.
// RM: K, dO, Out (OutCopy) and dQ are row-major head slices located by `ly`, V as well.
template <int WAVES, bool RM = false>
SPION_TILE_KERNEL(WAVES) void dense_bwd_row32_kernel(
    const float* __restrict__ Kt, const float* __restrict__ V, const float* __restrict__ Attn,
    const float* __restrict__ dOt, const float* __restrict__ OutCopy, float* __restrict__ G,
    float* __restrict__ dQ, int L, int nbr, int NB, float scale, Layouts ly) {
    constexpr int D = 32, KH = 16;
    __shared__ float lds[WAVES * 16 * 64];
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][3 * 1024];
    // last head first: the tail of the map is what the memory-side cache still holds after the forward
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = NB - 1 - item / nbr, I = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int nu = nbr > w ? (nbr - w + WAVES - 1) / WAVES : 0;
    const size_t hb = (size_t)bh * L * D;
    size_t ib, ob, gb, hbytes, obytes, gbytes;
    int ild, old_, gld;
    head_slice<RM, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<RM, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    head_slice<RM, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rdO = make_rsrc(dOt + ob, obytes);
    const char* Tv = reinterpret_cast<const char*>(lds_t[w]);
    const char* Tp = Tv + DmaTileF32::TILE;
    const char* Tk = Tv + 2 * DmaTileF32::TILE;

    float go[KH], oo[KH];
    if constexpr (RM) {
        ldr_rows<D>(rdO, (li * old_ + h * KH) * 4, I * 32 * old_ * 4, go);
        ldr_rows<D>(make_rsrc(OutCopy + ob, obytes), (li * old_ + h * KH) * 4, I * 32 * old_ * 4, oo);
    } else {
        ldr_cols<D>(rdO, L, (h * KH * L + li) * 4, I * 128, go);
        ldr_cols<D>(make_rsrc(OutCopy + hb, hbytes), L, (h * KH * L + li) * 4, I * 128, oo);
    }
    float g = 0.f;
#pragma unroll
    for (int s = 0; s < KH; ++s) g = fmaf(go[s], oo[s], g);
    g += __shfl_xor(g, 32, 64);
    if (w == 0 && h == 0) G[(size_t)bh * L + I * 32 + li] = -g;
    const f32x16 gneg = splat16(-g);

    f32x16 acc = splat16(0.f);  // dQ^T: register = feature, lane = query
    // The V, map and K tiles go straight into wave-private LDS; the operands of tile i are read out into registers,
    // then the same space is requested for tile i + 1, whose loads have the two chains of tile i to arrive.
    const unsigned lv = lds_address(Tv), lp = lv + DmaTileF32::TILE, lk = lv + 2 * DmaTileF32::TILE;
    const u32x4 wV = rsrc_words(V + ib, hbytes), wK = rsrc_words(Kt + ib, hbytes);
    const u32x4 wP = rsrc_words(Attn + (size_t)bh * L * L, (size_t)L * L * 4);
    const int kld = RM ? ild : L, KSTEP = RM ? 32 * ild * 4 : 128;
    const int vl = DmaTileF32::voff(l, ild), pl = DmaTileF32::voff(l, L), kl = DmaTileF32::voff(l, kld);
    const int vx = DmaTileF32::extra_step(ild), px = DmaTileF32::extra_step(L), kx = DmaTileF32::extra_step(kld);
    const auto a_v = DmaTileF32::own_addr(Tv, li, 4 * h, 1);  // V[key li][feature 16h + s]
    const auto a_p = DmaTileF32::cols_addr(Tp, li, h);        // P[query li][key acc_row(r, h)]
    const auto a_k = [&] {
        if constexpr (RM) return DmaTileF32::cols_addr(Tk, li, h);  // K^T[feature li][key acc_row(s, h)]
        else return DmaTileF32::own_addr(Tk, li, h, 2);
    }();
    auto issue = [&](int J) {
        DmaTileF32::load(wV, lv, vl, J * 32 * ild * 4, vx);
        DmaTileF32::load<true>(wP, lp, pl, (J * 32 * L + I * 32) * 4, px);
        DmaTileF32::load(wK, lk, kl, J * KSTEP, kx);
    };
    if (nu > 0) {
        issue(w);
        for (int i = 0; i < nu; ++i) {
            wait_vm<0>();
            float vt[16], pr[16], kb[16];
            DmaTileF32::get(a_v, vt);
            DmaTileF32::get(a_p, pr);
            DmaTileF32::get(a_k, kb);
            wait_lgkm0();
            if (i + 1 < nu) issue(w + (i + 1) * WAVES);
            __builtin_amdgcn_sched_barrier(0);
            f32x16 dp = mma_feat_init<D>(vt, go, gneg);  // register = key, lane = query: dO_i . v_j - g_i
            float ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = dp[r] * pr[r];
#pragma unroll
            for (int s = 0; s < 16; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(kb[s], ds[s], acc, 0, 0, 0);
        }
    }
    f32x16 out[1] = {acc * scale};
    if constexpr (RM) reduce_store_rows<WAVES>(out[0], dQ + gb, I * 32, w, li, h, lds, gld);
    else reduce_store<D, WAVES, true>(out, dQ + hb, I * 32, w, li, h, lds, L);
}

template <int WAVES, bool RM = false>
SPION_TILE_KERNEL(WAVES) void dense_bwd_col32_kernel(
    const float* __restrict__ Qt, const float* __restrict__ V, const float* __restrict__ Attn,
    const float* __restrict__ dOt, const float* __restrict__ G, float* __restrict__ dK, float* __restrict__ dV,
    int L, int nbr, int NB, float scale, Layouts ly) {
    constexpr int D = 32, KH = 16;
    __shared__ float lds[WAVES * 16 * 64];
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][3 * 1024 + 64];
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, J = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int nu = nbr > w ? (nbr - w + WAVES - 1) / WAVES : 0;
    const size_t hb = (size_t)bh * L * D;
    size_t ib, ob, gb, hbytes, obytes, gbytes;
    int ild, old_, gld;
    head_slice<RM, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<RM, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    head_slice<RM, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rV = make_rsrc(V + ib, hbytes);
    const char* To = reinterpret_cast<const char*>(lds_t[w]);
    const char* Tp = To + DmaTileF32::TILE;
    const char* Tq = To + 2 * DmaTileF32::TILE;
    const char* Tg = To + 3 * DmaTileF32::TILE;

    float v[KH];
    ldr_rows<D>(rV, (li * ild + h * KH) * 4, J * 32 * ild * 4, v);

    f32x16 ak = splat16(0.f), av = splat16(0.f);  // dK^T, dV^T: register = feature, lane = key
    // The dO, map and Q tiles and the 32 values of -g go straight into wave-private LDS; the operands of tile i are
    // read out into registers (the dO tile in both of its roles), then the same space is requested for tile i + 1.
    const unsigned lo = lds_address(To), lp = lo + DmaTileF32::TILE, lq = lo + 2 * DmaTileF32::TILE,
                   lg = lo + 3 * DmaTileF32::TILE;
    const u32x4 wO = rsrc_words(dOt + ob, obytes), wQ = rsrc_words(Qt + ib, hbytes);
    const u32x4 wP = rsrc_words(Attn + (size_t)bh * L * L, (size_t)L * L * 4), wG = rsrc_words(G + (size_t)bh * L, (size_t)L * 4);
    const int qld = RM ? ild : L, QSTEP = RM ? 32 * ild * 4 : 128;
    const int dld = RM ? old_ : L, DSTEP = RM ? 32 * old_ * 4 : 128;
    const int dl = DmaTileF32::voff(l, dld), pl = DmaTileF32::voff(l, L), ql = DmaTileF32::voff(l, qld);
    const int dx = DmaTileF32::extra_step(dld), px = DmaTileF32::extra_step(L), qx = DmaTileF32::extra_step(qld);
    const auto a_p = DmaTileF32::own_addr(Tp, li, h, 2);  // P[query acc_row(r, h)][key li]
    const char* a_g = Tg + 16 * h;                        // -g[query acc_row(r, h)]
    const auto a_go = [&] {
        if constexpr (RM) return DmaTileF32::own_addr(To, li, 4 * h, 1);  // dO[query li][feature 16h + s]
        else return DmaTileF32::featcols_addr(To, li, h);
    }();
    const auto a_qb = [&] {
        if constexpr (RM) return DmaTileF32::cols_addr(Tq, li, h);  // Q^T[feature li][query acc_row(s, h)]
        else return DmaTileF32::own_addr(Tq, li, h, 2);
    }();
    const auto a_ob = [&] {
        if constexpr (RM) return DmaTileF32::cols_addr(To, li, h);  // dO^T[feature li][query acc_row(s, h)]
        else return DmaTileF32::own_addr(To, li, h, 2);
    }();
    auto issue = [&](int I) {
        DmaTileF32::load(wO, lo, dl, I * DSTEP, dx);
        DmaTileF32::load<true>(wP, lp, pl, (J * 32 * L + I * 32) * 4, px);
        DmaTileF32::load(wQ, lq, ql, I * QSTEP, qx);
        dma_b32(wG, lg, l * 4, I * 128);
    };
    settle(v);
    if (nu > 0) {
        issue(w);
        for (int i = 0; i < nu; ++i) {
            wait_vm<0>();
            float go[16], ob[16], p[16], qb[16];
            f32x16 init;
            DmaTileF32::get(a_go, go);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 x = *reinterpret_cast<const f32x4*>(a_g + 32 * g);
                init[4 * g + 0] = x.x;
                init[4 * g + 1] = x.y;
                init[4 * g + 2] = x.z;
                init[4 * g + 3] = x.w;
            }
            DmaTileF32::get(a_p, p);
            DmaTileF32::get(a_qb, qb);
            DmaTileF32::get(a_ob, ob);
            wait_lgkm0();
            if (i + 1 < nu) issue(w + (i + 1) * WAVES);
            __builtin_amdgcn_sched_barrier(0);
            f32x16 dp = mma_feat_init<D>(go, v, init);  // register = query, lane = key
            float ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = dp[r] * p[r];
#pragma unroll
            for (int s = 0; s < 16; ++s) ak = __builtin_amdgcn_mfma_f32_32x32x2f32(qb[s], ds[s], ak, 0, 0, 0);
#pragma unroll
            for (int s = 0; s < 16; ++s) av = __builtin_amdgcn_mfma_f32_32x32x2f32(ob[s], p[s], av, 0, 0, 0);
        }
    }
    f32x16 out[1] = {ak * scale};
    if constexpr (RM) {
        reduce_store_rows<WAVES>(out[0], dK + gb, J * 32, w, li, h, lds, gld);
        __syncthreads();
        reduce_store_rows<WAVES>(av, dV + gb, J * 32, w, li, h, lds, gld);
        return;
    }
    reduce_store<D, WAVES, true>(out, dK + hb, J * 32, w, li, h, lds, L);
    __syncthreads();
    out[0] = av;
    reduce_store<D, WAVES, true>(out, dV + hb, J * 32, w, li, h, lds, L);
}

// Backward passes for d = 64, row-major operands (the strided entry points): the d = 64 schedule of the sparse tile
// kernels (tile_kernels.h) on the dense map.  A wavefront's LDS holds five 4 KB tiles -- the map tile and two
// 32-feature halves each of the two operand tiles -- 20 KB, so that four wavefronts take 80 KB and two work-groups
// fill a CU to the last byte; the buffer of the final reduction lies inside the tile space, a barrier in between.
template <int WAVES>
SPION_TILE_KERNEL(WAVES) void dense_bwd_row64_kernel(
    const float* __restrict__ K, const float* __restrict__ V, const float* __restrict__ Attn,
    const float* __restrict__ dO, const float* __restrict__ Out, float* __restrict__ G, float* __restrict__ dQ,
    int L, int nbr, int NB, float scale, Layouts ly) {
    constexpr int D = 64, KH = 32, WB = 5 * DmaTileF32::TILE;
    static_assert(WAVES * 2 * 16 * 64 * 4 <= WAVES * WB, "the reduction fits in the tile space");
    __shared__ __attribute__((aligned(16))) char smem[WAVES * WB];
    // last head first: the tail of the map is what the memory-side cache still holds after the forward
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = NB - 1 - item / nbr, I = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int nu = nbr > w ? (nbr - w + WAVES - 1) / WAVES : 0;
    size_t ib, ob, gb, hbytes, obytes, gbytes;
    int ild, old_, gld;
    head_slice<true, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<true, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    head_slice<true, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);

    float go[KH], oo[KH];
    ldr_rows<D>(make_rsrc(dO + ob, obytes), (li * old_ + h * KH) * 4, I * 32 * old_ * 4, go);
    ldr_rows<D>(make_rsrc(Out + ob, obytes), (li * old_ + h * KH) * 4, I * 32 * old_ * 4, oo);
    float g = 0.f;
#pragma unroll
    for (int s = 0; s < KH; ++s) g = fmaf(go[s], oo[s], g);
    g += __shfl_xor(g, 32, 64);
    if (w == 0 && h == 0) G[(size_t)bh * L + I * 32 + li] = -g;
    const f32x16 gneg = splat16(-g);

    f32x16 acc[2] = {splat16(0.f), splat16(0.f)};  // dQ: register = query, lane = feature
    const char* Tv = smem + w * WB;
    const char* Tk = Tv + 2 * DmaTileF32::TILE;
    const char* Tp = Tv + 4 * DmaTileF32::TILE;
    const unsigned lv = lds_address(Tv), lk = lv + 2 * DmaTileF32::TILE, lp = lv + 4 * DmaTileF32::TILE;
    const u32x4 wV = rsrc_words(V + ib, hbytes), wK = rsrc_words(K + ib, hbytes);
    const u32x4 wP = rsrc_words(Attn + (size_t)bh * L * L, (size_t)L * L * 4);
    const int vl = DmaTileF32::voff(l, ild), pl = DmaTileF32::voff(l, L);
    const int vx = DmaTileF32::extra_step(ild), px = DmaTileF32::extra_step(L);
    const auto a_v = DmaTileF32::own8_addr(Tv + h * DmaTileF32::TILE, li);  // V[key li][feature 32h + s]
    const auto a_p = DmaTileF32::cols_addr(Tp, li, h);                      // P[query li][key acc_row(r, h)]
    const auto a_k = DmaTileF32::cols_addr(Tk, li, h);                      // K[key acc_row(s, h)][feature li (+32)]
    auto issue = [&](int J) {
        DmaTileF32::load(wV, lv, vl, J * 32 * ild * 4, vx);
        DmaTileF32::load(wV, lv + DmaTileF32::TILE, vl, J * 32 * ild * 4 + 128, vx);
        DmaTileF32::load<true>(wP, lp, pl, (J * 32 * L + I * 32) * 4, px);
        DmaTileF32::load(wK, lk, vl, J * 32 * ild * 4, vx);
        DmaTileF32::load(wK, lk + DmaTileF32::TILE, vl, J * 32 * ild * 4 + 128, vx);
    };
    if (nu > 0) {
        issue(w);
        for (int i = 0; i < nu; ++i) {
            wait_vm<0>();
            float vt[KH], pr[16], kb[2][16];
            DmaTileF32::get32(a_v, vt);
            DmaTileF32::get(a_p, pr);
            DmaTileF32::get(a_k, kb[0]);
            DmaTileF32::get(a_k, kb[1], DmaTileF32::TILE);
            wait_lgkm0();
            if (i + 1 < nu) issue(w + (i + 1) * WAVES);
            __builtin_amdgcn_sched_barrier(0);
            f32x16 dp = mma_feat_init<D>(vt, go, gneg);  // register = key, lane = query: dO_i . v_j - g_i
            float ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = dp[r] * pr[r];
            mma_b<D>(ds, kb, acc);
        }
    }
    if (WAVES > 1) __syncthreads();  // every wavefront is done with its tiles
    acc[0] *= scale;
    acc[1] *= scale;
    reduce_store<D, WAVES>(acc, dQ + gb, I * 32, w, li, h, reinterpret_cast<float*>(smem), gld);
}

// -g does not fit beside the tiles: each lane loads the value of query row lane % 32 of the next tile with an ordinary
// load, and one extra MFMA step -- A = that value in the lower half-wave, zero in the upper, B = 1 -- spreads it over
// the accumulator the dP chain starts from.
template <int WAVES>
SPION_TILE_KERNEL(WAVES) void dense_bwd_col64_kernel(
    const float* __restrict__ Q, const float* __restrict__ V, const float* __restrict__ Attn,
    const float* __restrict__ dO, const float* __restrict__ G, float* __restrict__ dK, float* __restrict__ dV,
    int L, int nbr, int NB, float scale, Layouts ly) {
    constexpr int D = 64, KH = 32, WB = 5 * DmaTileF32::TILE;
    static_assert(WAVES * 2 * 16 * 64 * 4 <= WAVES * WB, "the reduction fits in the tile space");
    __shared__ __attribute__((aligned(16))) char smem[WAVES * WB];
    const int item = xcd_remap(blockIdx.x, nbr * NB);
    const int bh = item / nbr, J = item % nbr;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int nu = nbr > w ? (nbr - w + WAVES - 1) / WAVES : 0;
    size_t ib, ob, gb, hbytes, obytes, gbytes;
    int ild, old_, gld;
    head_slice<true, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<true, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    head_slice<true, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rG = make_rsrc(G + (size_t)bh * L, (size_t)L * 4);

    float vt[KH];
    ldr_rows<D>(make_rsrc(V + ib, hbytes), (li * ild + h * KH) * 4, J * 32 * ild * 4, vt);

    f32x16 ak[2] = {splat16(0.f), splat16(0.f)}, av[2] = {splat16(0.f), splat16(0.f)};  // register = key, lane = feature
    const char* Tp = smem + w * WB;
    const char* Tq = Tp + DmaTileF32::TILE;
    const char* To = Tp + 3 * DmaTileF32::TILE;
    const unsigned lp = lds_address(Tp), lq = lp + DmaTileF32::TILE, lo = lp + 3 * DmaTileF32::TILE;
    const u32x4 wQ = rsrc_words(Q + ib, hbytes), wO = rsrc_words(dO + ob, obytes);
    const u32x4 wP = rsrc_words(Attn + (size_t)bh * L * L, (size_t)L * L * 4);
    const int ql = DmaTileF32::voff(l, ild), ol = DmaTileF32::voff(l, old_), pl = DmaTileF32::voff(l, L);
    const int qx = DmaTileF32::extra_step(ild), ox = DmaTileF32::extra_step(old_), px = DmaTileF32::extra_step(L);
    const auto a_p = DmaTileF32::own_addr(Tp, li, h, 2);  // P[query acc_row(r, h)][key li]
    const auto a_q = DmaTileF32::cols_addr(Tq, li, h);    // Q[query acc_row(s, h)][feature li (+32)]
    const auto a_o = DmaTileF32::cols_addr(To, li, h);    // dO[query acc_row(s, h)][feature li (+32)]
    const auto a_go = DmaTileF32::own8_addr(To + h * DmaTileF32::TILE, li);  // dO[query li][feature 32h + s]
    auto issue = [&](int I) {
        DmaTileF32::load<true>(wP, lp, pl, (J * 32 * L + I * 32) * 4, px);
        DmaTileF32::load(wQ, lq, ql, I * 32 * ild * 4, qx);
        DmaTileF32::load(wQ, lq + DmaTileF32::TILE, ql, I * 32 * ild * 4 + 128, qx);
        DmaTileF32::load(wO, lo, ol, I * 32 * old_ * 4, ox);
        DmaTileF32::load(wO, lo + DmaTileF32::TILE, ol, I * 32 * old_ * 4 + 128, ox);
    };
    settle(vt);
    if (nu > 0) {
        issue(w);
        float gl = ld1(rG, li * 4, w * 128);
        for (int i = 0; i < nu; ++i) {
            wait_vm<0>();
            settle(gl);
            const float ga = h == 0 ? gl : 0.f;
            float pc[16], qb[2][16], ob[2][16], go[KH];
            DmaTileF32::get32(a_go, go);
            DmaTileF32::get(a_p, pc);
            DmaTileF32::get(a_q, qb[0]);
            DmaTileF32::get(a_q, qb[1], DmaTileF32::TILE);
            DmaTileF32::get(a_o, ob[0]);
            DmaTileF32::get(a_o, ob[1], DmaTileF32::TILE);
            wait_lgkm0();
            if (i + 1 < nu) {
                issue(w + (i + 1) * WAVES);
                gl = ld1(rG, li * 4, (w + (i + 1) * WAVES) * 128);
            }
            __builtin_amdgcn_sched_barrier(0);
            const f32x16 init = __builtin_amdgcn_mfma_f32_32x32x2f32(ga, 1.0f, splat16(0.f), 0, 0, 0);  // -g_i in every column
            f32x16 dp = mma_feat_init<D>(go, vt, init);  // register = query, lane = key
            float ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = dp[r] * pc[r];
            mma_b<D>(ds, qb, ak);
            mma_b<D>(pc, ob, av);
        }
    }
    if (WAVES > 1) __syncthreads();  // every wavefront is done with its tiles
    ak[0] *= scale;
    ak[1] *= scale;
    reduce_store<D, WAVES>(ak, dK + gb, J * 32, w, li, h, reinterpret_cast<float*>(smem), gld);
    if (WAVES > 1) __syncthreads();
    reduce_store<D, WAVES>(av, dV + gb, J * 32, w, li, h, reinterpret_cast<float*>(smem), gld);
}

// -------------------------------------------------------------------------------------------------
struct DenseAttn {
    HandleHeader hdr;
    int d, L, NB;
    bool has_mask;
    float scale;
    float* ws_rowsum = nullptr;  // [NB][L]
    // Copy of Out kept by the forward, filed under the map (Attn) it filled: a backward handed the same map
    // takes its row sums g_i = dO_i . O_i from it instead of a sweep over the whole map.
    float* ws_out = nullptr;      // [NB][d][L]
    const float* out_key = nullptr;
    float* ws_mean = nullptr;     // [C][L][L] partial sums of the maps (mean-emitting forward)
    size_t ws_mean_floats = 0;
};

static DenseAttn* as_dense(void* h, const char* who) {
    DenseAttn* a = static_cast<DenseAttn*>(h);
    note_current_handle(a && a->hdr.magic == KIND_DENSE ? &a->hdr : nullptr);
    if (!a || a->hdr.magic != KIND_DENSE) {
        set_error("%s: not a dense-attention handle", who);
        return nullptr;
    }
    return a;
}

void* dense_init(int emb_dim, int seq_len, int num_batches, bool has_mask) {
    if (seq_len <= 0 || num_batches <= 0 || seq_len % 32) {
        set_error("dense init: seq_len must be a positive multiple of 32 and num_batches positive (got %d, %d)",
                  seq_len, num_batches);
        return nullptr;
    }
    if (emb_dim != 32 && emb_dim != 64) {
        set_error("dense init: emb_dim %d unsupported (32 or 64)", emb_dim);
        return nullptr;
    }
    DenseAttn* a = new DenseAttn();
    a->hdr.magic = KIND_DENSE;
    a->hdr.stream = nullptr;
    a->hdr.err[0] = 0;
    a->d = emb_dim;
    a->L = seq_len;
    a->NB = num_batches;
    a->has_mask = has_mask;
    a->scale = 1.0f / sqrtf((float)emb_dim);  // models/attn.cu:153
    return a;
}

void dense_destroy(void* h) {
    DenseAttn* a = as_dense(h, "destroy");
    if (!a) return;
    if (a->ws_rowsum) (void)hipFree(a->ws_rowsum);
    if (a->ws_out) (void)hipFree(a->ws_out);
    if (a->ws_mean) (void)hipFree(a->ws_mean);
    a->hdr.magic = 0;
    note_current_handle(nullptr);
    delete a;
}

template <int D>
static void dense_fwd_launch(DenseAttn* a, const float* Qt, const float* K, const float* Vt, const float* Mask,
                             float* Attn, float* Out) {
    const int nbr = a->L / 32;
    dim3 grid(nbr * a->NB), block(64 * DENSE_WAVES);
    if (!a->ws_out && hipMalloc((void**)&a->ws_out, sizeof(float) * (size_t)a->NB * a->L * a->d) != hipSuccess) {
        (void)hipGetLastError();  // no copy: the backward sweeps the map for its row sums
        a->ws_out = nullptr;
    }
    a->out_key = a->ws_out ? Attn : nullptr;
    if (D == 32 && nbr <= 32) {
        const dim3 block4(64 * 4);
        if (a->has_mask)
            hipLaunchKernelGGL(dense_fwd_reg_kernel<true>, grid, block4, 0, a->hdr.stream, Qt, K, Vt, Mask, Attn, Out,
                               a->ws_out, a->L, nbr, a->NB, a->scale, Layouts{});
        else
            hipLaunchKernelGGL(dense_fwd_reg_kernel<false>, grid, block4, 0, a->hdr.stream, Qt, K, Vt, Mask, Attn, Out,
                               a->ws_out, a->L, nbr, a->NB, a->scale, Layouts{});
        return;
    }
    if (D == 32 && nbr <= 64) {  // eight wavefronts with at most eight logit tiles each
        const dim3 block8(64 * 8);
        if (a->has_mask)
            hipLaunchKernelGGL((dense_fwd_reg_kernel<true, false, 8, false, 8>), grid, block8, 0, a->hdr.stream, Qt, K, Vt,
                               Mask, Attn, Out, a->ws_out, a->L, nbr, a->NB, a->scale, Layouts{});
        else
            hipLaunchKernelGGL((dense_fwd_reg_kernel<false, false, 8, false, 8>), grid, block8, 0, a->hdr.stream, Qt, K, Vt,
                               Mask, Attn, Out, a->ws_out, a->L, nbr, a->NB, a->scale, Layouts{});
        return;
    }
    if (D == 32 && a->L <= 16384) {  // 32-bit byte offsets into one head's map: L*L*4 < 2^31
        const dim3 block4(64 * 4);
        if (a->has_mask)
            hipLaunchKernelGGL(dense_fwd_sweep32_kernel<true>, grid, block4, 0, a->hdr.stream, Qt, K, Vt, Mask, Attn,
                               Out, a->ws_out, a->L, nbr, a->NB, a->scale, Layouts{});
        else
            hipLaunchKernelGGL(dense_fwd_sweep32_kernel<false>, grid, block4, 0, a->hdr.stream, Qt, K, Vt, Mask, Attn,
                               Out, a->ws_out, a->L, nbr, a->NB, a->scale, Layouts{});
        return;
    }
    if (a->has_mask)
        hipLaunchKernelGGL((dense_fwd_kernel<D, true>), grid, block, 0, a->hdr.stream, Qt, K, Vt, Mask, Attn, Out,
                           a->ws_out, a->L, nbr, a->NB, a->scale);
    else
        hipLaunchKernelGGL((dense_fwd_kernel<D, false>), grid, block, 0, a->hdr.stream, Qt, K, Vt, Mask, Attn, Out,
                           a->ws_out, a->L, nbr, a->NB, a->scale);
}

template <int D>
static void dense_bwd_launch(DenseAttn* a, const float* Qt, const float* Kt, const float* V, const float* P,
                             const float* dOt, float* dQ, float* dK, float* dV) {
    const int nbr = a->L / 32;
    dim3 grid(nbr * a->NB), block(64 * DENSE_WAVES);
    // 32-bit byte offsets into one head's map: L*L*4 < 2^31
    if (D == 32 && a->L <= 16384 && a->out_key == P && a->ws_out) {
        const dim3 block4(64 * 4);
        hipLaunchKernelGGL(dense_bwd_row32_kernel<4>, grid, block4, 0, a->hdr.stream, Kt, V, P, dOt, a->ws_out,
                           a->ws_rowsum, dQ, a->L, nbr, a->NB, a->scale, Layouts{});
        hipLaunchKernelGGL(dense_bwd_col32_kernel<4>, grid, block4, 0, a->hdr.stream, Qt, V, P, dOt, a->ws_rowsum, dK,
                           dV, a->L, nbr, a->NB, a->scale, Layouts{});
        return;
    }
    if (a->out_key == P && a->ws_out)
        hipLaunchKernelGGL((dense_bwd_row_kernel<D, true>), grid, block, 0, a->hdr.stream, Kt, V, P, dOt, a->ws_out,
                           a->ws_rowsum, dQ, a->L, nbr, a->NB, a->scale);
    else
        hipLaunchKernelGGL((dense_bwd_row_kernel<D, false>), grid, block, 0, a->hdr.stream, Kt, V, P, dOt, a->ws_out,
                           a->ws_rowsum, dQ, a->L, nbr, a->NB, a->scale);
    hipLaunchKernelGGL((dense_bwd_col_kernel<D>), grid, block, 0, a->hdr.stream, Qt, V, P, dOt, a->ws_rowsum, dK, dV,
                       a->L, nbr, a->NB, a->scale);
}

void dense_forward(void* h, const float* Qt, const float* K, const float* Vt, const float* Mask, float* Attn,
                   float* Out, bool mask_entry) {
    DenseAttn* a = as_dense(h, "attn_forward");
    if (!a) return;
    if (a->has_mask != mask_entry) {
        set_error("attn_forward: handle was created by the %s init", a->has_mask ? "mask" : "no-mask");
        return;
    }
    if (!Qt || !K || !Vt || !Attn || !Out || (mask_entry && !Mask)) {
        set_error("attn_forward: null pointer argument");
        return;
    }
    if (a->d == 32) dense_fwd_launch<32>(a, Qt, K, Vt, Mask, Attn, Out);
    else dense_fwd_launch<64>(a, Qt, K, Vt, Mask, Attn, Out);
    check_launch("dense_fwd_kernel");
}

void dense_backward(void* h, const float* Qt, const float* Kt, const float* V, const float* P, const float* dOt,
                    float* dQ, float* dK, float* dV) {
    DenseAttn* a = as_dense(h, "attn_backward");
    if (!a) return;
    if (!Qt || !Kt || !V || !P || !dOt || !dQ || !dK || !dV) {
        set_error("attn_backward: null pointer argument");
        return;
    }
    if (!a->ws_rowsum && !SPION_HIP_OK(hipMalloc((void**)&a->ws_rowsum, sizeof(float) * (size_t)a->NB * a->L))) return;
    if (a->d == 32) dense_bwd_launch<32>(a, Qt, Kt, V, P, dOt, dQ, dK, dV);
    else dense_bwd_launch<64>(a, Qt, Kt, V, P, dOt, dQ, dK, dV);
    check_launch("dense_bwd kernels");
}

// Row-major / strided heads (L <= 16384; d = 64: the forward for L <= 2048 only): Q, K, V, Out, dO and the gradients
// are [B][H][L][d] views with one layout per tensor group (tile_kernels.h), read and written in place; the map stays
// [NB][key][query].
static DenseAttn* dense_strided_handle(void* h, const char* who, int heads, const HeadLayout* const* lays, int n) {
    DenseAttn* a = as_dense(h, who);
    if (!a) return nullptr;
    if (a->L > 16384) {  // 32-bit byte offsets into one head's map: L*L*4 < 2^31
        set_error("%s: strided heads are served for seq_len <= 16384 only", who);
        return nullptr;
    }
    if (heads <= 0 || a->NB % heads) {
        set_error("%s: heads = %d does not divide num_batches = %d", who, heads, a->NB);
        return nullptr;
    }
    for (int i = 0; i < n; ++i) {
        const HeadLayout& y = *lays[i];
        if (y.ld < a->d || y.ld % 4 || y.hstride % 4 || y.bstride % 4 || y.hstride < 0 || y.bstride < 0 ||
            (long long)a->L * y.ld >= (1ll << 29)) {
            set_error("%s: layout %d: strides must be non-negative multiples of 4 floats, row stride >= emb_dim, "
                      "seq_len * row stride < 2^29", who, i);
            return nullptr;
        }
    }
    return a;
}
static bool dense_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int score_map_mean(const float* Attn, int batch, int heads, int L, int key_major, float* Mean, hipStream_t stream,
                   float post);

// Mean != nullptr: the launch also leaves the mean of all NB maps (queries x keys) in Mean, accumulated while the
// maps are written (see dense_fwd_reg_kernel) and finished by one reduction over the partial maps.
static void dense_forward_strided_impl(void* h, const float* Q, const float* K, const float* V, const float* Mask,
                                       float* Attn, float* Out, float* Mean, int heads, const HeadLayout& in,
                                       const HeadLayout& out, const char* who) {
    const HeadLayout* lays[2] = {&in, &out};
    DenseAttn* a = dense_strided_handle(h, who, heads, lays, 2);
    if (!a) return;
    if (a->has_mask != (Mask != nullptr)) {
        set_error("%s: handle was created by the %s init", who, a->has_mask ? "mask" : "no-mask");
        return;
    }
    if (!Q || !K || !V || !Attn || !Out) {
        set_error("%s: null pointer argument", who);
        return;
    }
    if (!dense_aligned16(Q) || !dense_aligned16(K) || !dense_aligned16(V) || !dense_aligned16(Out)) {
        set_error("%s: operand pointers must be 16-byte aligned", who);
        return;
    }
    if (!layout_is_injective(out, a->NB / heads, heads, a->L, a->d)) {
        set_error("%s: the output layout maps two elements to one address", who);
        return;
    }
    Layouts ly{};
    ly.in = in;
    ly.out = out;
    ly.grad = out;
    ly.H = heads;
    const int nbr = a->L / 32;
    const dim3 grid(nbr * a->NB), block4(64 * 4);
    a->out_key = nullptr;  // no kept copy: the strided backward is handed Out
    if (a->d == 64) {
        if (Mean || nbr > 64) {
            set_error("%s: emb_dim 64 is served for seq_len <= 2048 and without the mean map", who);
            return;
        }
        // at most eight logit tiles per wavefront: four wavefronts up to L = 1024, eight up to 2048
#define SPION_LAUNCH(MM, W)                                                                                          \
    hipLaunchKernelGGL((dense_fwd_reg64_kernel<MM, W>), grid, dim3(64 * W), 0, a->hdr.stream, Q, K, V, Mask, Attn, Out, \
                       a->L, nbr, a->NB, a->scale, ly)
        if (nbr <= 32) {
            if (a->has_mask) SPION_LAUNCH(true, 4);
            else SPION_LAUNCH(false, 4);
        } else {
            if (a->has_mask) SPION_LAUNCH(true, 8);
            else SPION_LAUNCH(false, 8);
        }
#undef SPION_LAUNCH
        check_launch("dense_fwd kernels");
        return;
    }
    if (Mean) {
        // C partial maps: the smallest divisor of NB that fills the device -- one eight-wavefront work-group per CU
        // for the register-resident form (measured at B=256, H=2, L=1024: 0.95 ms with 256 work-groups, 1.05 with
        // 512, 1.22 with 1024: fewer, longer work-groups store fewer partial maps), two four-wavefront ones otherwise
        static int cus = 0;
        if (!cus) {
            int dev = 0;
            if (hipGetDevice(&dev) != hipSuccess ||
                hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
                (void)hipGetLastError();
                cus = 256;
            }
        }
        const long long want = nbr <= 32 ? cus : 2LL * cus;
        int C = a->NB;
        for (int c = 1; c <= a->NB; ++c)
            if (a->NB % c == 0 && (long long)c * nbr >= want) {
                C = c;
                break;
            }
        // C follows from the handle's shape alone, so the partial maps are allocated once per handle and their
        // address never changes afterwards (a recorded HIP graph stays valid); never under capture, where an
        // allocation would invalidate the capture
        const size_t need = (size_t)C * a->L * a->L;
        if (need > a->ws_mean_floats) {
            hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
            (void)hipStreamIsCapturing(a->hdr.stream, &cap);
            if (cap != hipStreamCaptureStatusNone || a->ws_mean) {
                set_error("%s: the partial maps are not allocated yet; run one call outside the capture", who);
                return;
            }
            if (!SPION_HIP_OK(hipMalloc((void**)&a->ws_mean, sizeof(float) * need))) return;
            a->ws_mean_floats = need;
        }
        const dim3 grid_m(nbr * C);
#define SPION_LAUNCH(KERNEL, MM)                                                                                     \
    hipLaunchKernelGGL((KERNEL<MM, true, true>), grid_m, block4, 0, a->hdr.stream, Q, K, V, Mask, Attn, Out, nullptr, \
                       a->L, nbr, a->NB, a->scale, ly, a->ws_mean, C)
        if (nbr <= 32) {
            // register-resident logits on eight wavefronts, the partial sums in registers as well
            const dim3 block8(64 * 8);
            if (a->has_mask)
                hipLaunchKernelGGL((dense_fwd_reg_kernel<true, true, 8, true>), grid_m, block8, 0, a->hdr.stream, Q, K, V,
                                   Mask, Attn, Out, nullptr, a->L, nbr, a->NB, a->scale, ly, a->ws_mean, C);
            else
                hipLaunchKernelGGL((dense_fwd_reg_kernel<false, true, 8, true>), grid_m, block8, 0, a->hdr.stream, Q, K, V,
                                   Mask, Attn, Out, nullptr, a->L, nbr, a->NB, a->scale, ly, a->ws_mean, C);
        } else if (a->has_mask) SPION_LAUNCH(dense_fwd_sweep32_kernel, true);
        else SPION_LAUNCH(dense_fwd_sweep32_kernel, false);
#undef SPION_LAUNCH
        if (!check_launch("dense_fwd kernels")) return;
        // mean over the C partial sums, times C / NB: the mean of all maps, transposed to queries x keys
        (void)score_map_mean(a->ws_mean, C, 1, a->L, 1, Mean, a->hdr.stream, (float)C / (float)a->NB);
        return;
    }
    if (nbr <= 32) {
        if (a->has_mask)
            hipLaunchKernelGGL((dense_fwd_reg_kernel<true, true>), grid, block4, 0, a->hdr.stream, Q, K, V, Mask, Attn,
                               Out, nullptr, a->L, nbr, a->NB, a->scale, ly);
        else
            hipLaunchKernelGGL((dense_fwd_reg_kernel<false, true>), grid, block4, 0, a->hdr.stream, Q, K, V, Mask, Attn,
                               Out, nullptr, a->L, nbr, a->NB, a->scale, ly);
    } else if (nbr <= 64) {  // eight wavefronts with at most eight logit tiles each
        const dim3 block8(64 * 8);
        if (a->has_mask)
            hipLaunchKernelGGL((dense_fwd_reg_kernel<true, true, 8, false, 8>), grid, block8, 0, a->hdr.stream, Q, K, V,
                               Mask, Attn, Out, nullptr, a->L, nbr, a->NB, a->scale, ly);
        else
            hipLaunchKernelGGL((dense_fwd_reg_kernel<false, true, 8, false, 8>), grid, block8, 0, a->hdr.stream, Q, K, V,
                               Mask, Attn, Out, nullptr, a->L, nbr, a->NB, a->scale, ly);
    } else {
        if (a->has_mask)
            hipLaunchKernelGGL((dense_fwd_sweep32_kernel<true, true>), grid, block4, 0, a->hdr.stream, Q, K, V, Mask,
                               Attn, Out, nullptr, a->L, nbr, a->NB, a->scale, ly);
        else
            hipLaunchKernelGGL((dense_fwd_sweep32_kernel<false, true>), grid, block4, 0, a->hdr.stream, Q, K, V, Mask,
                               Attn, Out, nullptr, a->L, nbr, a->NB, a->scale, ly);
    }
    check_launch("dense_fwd kernels");
}

void dense_forward_strided(void* h, const float* Q, const float* K, const float* V, const float* Mask, float* Attn,
                           float* Out, int heads, const HeadLayout& in, const HeadLayout& out) {
    dense_forward_strided_impl(h, Q, K, V, Mask, Attn, Out, nullptr, heads, in, out, "dense attn_forward_strided");
}
void dense_forward_strided_mean(void* h, const float* Q, const float* K, const float* V, const float* Mask, float* Attn,
                                float* Out, float* Mean, int heads, const HeadLayout& in, const HeadLayout& out) {
    if (!Mean) {
        as_dense(h, "dense attn_forward_strided_mean");
        set_error("dense attn_forward_strided_mean: null Mean");
        return;
    }
    dense_forward_strided_impl(h, Q, K, V, Mask, Attn, Out, Mean, heads, in, out, "dense attn_forward_strided_mean");
}

void dense_backward_strided(void* h, const float* Q, const float* K, const float* V, const float* P, const float* Out,
                            const float* dO, float* dQ, float* dK, float* dV, int heads, const HeadLayout& in,
                            const HeadLayout& out, const HeadLayout& grad) {
    const char* who = "dense attn_backward_strided";
    const HeadLayout* lays[3] = {&in, &out, &grad};
    DenseAttn* a = dense_strided_handle(h, who, heads, lays, 3);
    if (!a) return;
    if (!Q || !K || !V || !P || !Out || !dO || !dQ || !dK || !dV) {
        set_error("%s: null pointer argument", who);
        return;
    }
    if (!dense_aligned16(Q) || !dense_aligned16(K) || !dense_aligned16(V) || !dense_aligned16(Out) ||
        !dense_aligned16(dO) || !dense_aligned16(dQ) || !dense_aligned16(dK) || !dense_aligned16(dV)) {
        set_error("%s: operand pointers must be 16-byte aligned", who);
        return;
    }
    if (!layout_is_injective(grad, a->NB / heads, heads, a->L, a->d)) {
        set_error("%s: the gradient layout maps two elements to one address", who);
        return;
    }
    if (!a->ws_rowsum && !SPION_HIP_OK(hipMalloc((void**)&a->ws_rowsum, sizeof(float) * (size_t)a->NB * a->L))) return;
    Layouts ly{};
    ly.in = in;
    ly.out = out;
    ly.grad = grad;
    ly.H = heads;
    const int nbr = a->L / 32;
    const dim3 grid(nbr * a->NB), block4(64 * 4);
    if (a->d == 64) {
        hipLaunchKernelGGL(dense_bwd_row64_kernel<4>, grid, block4, 0, a->hdr.stream, K, V, P, dO, Out, a->ws_rowsum,
                           dQ, a->L, nbr, a->NB, a->scale, ly);
        hipLaunchKernelGGL(dense_bwd_col64_kernel<4>, grid, block4, 0, a->hdr.stream, Q, V, P, dO, a->ws_rowsum, dK, dV,
                           a->L, nbr, a->NB, a->scale, ly);
    } else {
        hipLaunchKernelGGL((dense_bwd_row32_kernel<4, true>), grid, block4, 0, a->hdr.stream, K, V, P, dO, Out,
                           a->ws_rowsum, dQ, a->L, nbr, a->NB, a->scale, ly);
        hipLaunchKernelGGL((dense_bwd_col32_kernel<4, true>), grid, block4, 0, a->hdr.stream, Q, V, P, dO, a->ws_rowsum,
                           dK, dV, a->L, nbr, a->NB, a->scale, ly);
    }
    check_launch("dense_bwd kernels");
}

}  // namespace spion
