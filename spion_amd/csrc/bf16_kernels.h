// bf16 tile kernels of the sparse path (scale-up configuration: bf16 tensors, fp32 accumulation and softmax).
//
// No counterpart in the reference (fp32 only); the semantics are those of models/block_attn.cu:33-130 (and
// the key-penalty variant models/block_attn_mask.cu:88-173) with the probabilities never written to memory:
// the forward stores one fp32 number per row, lse2_i = m_i + log2(Z_i) in the log2 domain, and both
// backward passes recompute P_ij = exp2(s_ij*log2(e)/sqrt(d) - lse2_i) from Q and K.
//
// All tensors are row-major [head][L][D] bf16.  Every contraction is a chain of v_mfma_f32_32x32x16_bf16
// (lane l supplies 8 consecutive k-slots of row l%32 for both operands, half-wave l/32 the second 8; the
// fp32 accumulator layout is the one of every 32x32 MFMA: register r of lane l is row acc_row(r, l/32),
// column l%32).  Which feature / tile row a k-slot stands for is free as long as both operands agree:
//   * products over the head dimension: lane (row, h) holds features h*D/2 .. h*D/2+D/2-1 of its row, D/2
//     consecutive bf16 of a row-major row (D/16 instructions);
//   * products over a tile's 32 keys or queries: slot e of instruction t in half h is tile row
//     16t + 8(e/4) + 4h + e%4 = acc_row(8t+e, h), so the accumulator of the first product, converted to
//     bf16, is the B operand of the second one register for register.  The A operand (the tile of K, V, Q or
//     dO seen feature-major) is read from the tile's wave-private LDS copy with the transposing LDS read
//     of gfx950.
// Tiles travel global memory -> wave-private LDS buffers (buffer loads with the LDS modifier, two tiles ahead) ->
// operand layouts; same-wave LDS accesses complete in order, so no barrier is involved.
// Queries are the lane index of every row-pass accumulator (S^T, dP^T, O^T, dQ^T), so row statistics are
// lane scalars; keys are the lane index in the column pass.
//
// A launch is a fixed set of persistent one-wavefront work-groups, two per SIMD, each walking a host-built list of
// items: whole strips, pairs of strips (forward) or chunks of a long strip (a global row or column, cut so that it
// does not outlast the rest of the launch; every chunk leaves fp32 partial results in a workspace slot and a small
// merge kernel combines the slots of a strip).
#pragma once
#include "tile_kernels.h"

namespace spion {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

constexpr float BF16_LAZY = 8.f;  // the running row maximum is raised only when a tile exceeds it by 2^8

template <int D>
__device__ __forceinline__ void ldb_rows(rsrc_t r, int voff, int soff, bf16x8 (&x)[D / 16]) {
#pragma unroll
    for (int t = 0; t < D / 16; ++t)
        x[t] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff + 16 * t, 0));
}

// Start (in elements), row stride and size in bytes of head bh: contiguous [NB][L][D] heads (ST = false, compile-time
// figures) or [B][H][L][D] views given by a layout (strides in elements).
template <bool ST, int D>
__device__ __forceinline__ void bf16_head(const HeadLayout& y, int H, int bh, int L, size_t& base, int& ld,
                                          size_t& bytes) {
    head_slice<ST, D>(y, H, bh, L, base, ld, bytes);
    bytes >>= 1;  // head_slice counts four bytes an element
}

template <int D>
__device__ __forceinline__ f32x16 mma_feat_bf16(const bf16x8 (&a)[D / 16], const bf16x8 (&b)[D / 16], f32x16 init) {
    f32x16 acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[0], init, 0, 0, 0);
#pragma unroll
    for (int t = 1; t < D / 16; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[t], b[t], acc, 0, 0, 0);
    return acc;
}

// out[c] (features 32c.. x lanes) += X_tile^T . W^T, W given as accumulator-layout values packed to bf16
template <int D>
__device__ __forceinline__ void mma_tile_bf16(const bf16x8 (&xt)[D / 32][2], const bf16x8 (&wb)[2], f32x16 (&out)[D / 32]) {
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
#pragma unroll
        for (int t = 0; t < 2; ++t) out[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xt[c][t], wb[t], out[c], 0, 0, 0);
}

__device__ __forceinline__ void pack16(const float (&p)[16], bf16x8 (&pb)[2]) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[t][e] = (__bf16)p[8 * t + e];
}

// -------------------------------------------------------------------------------------------------
// Tiles that go from global memory straight into LDS (buffer loads with the LDS modifier): no registers hold a
// tile in flight and no ds_write is spent on it.  One instruction moves 64 x 16 bytes to 1 KB of consecutive LDS
// addresses starting at M0 (+ the instruction's immediate offset, which is added to the global address as well);
// which 16-byte piece of global memory a lane fetches is free, so the LDS image of a tile is unpadded rows with
// the pieces of a row permuted: piece c of tile row r lies at position c ^ swz(r).  With that permutation the
// transposing reads (four consecutive rows of two adjacent pieces, thirty-two lanes at a time) are free of bank
// conflicts; the 16-byte reads of an operand over the head dimension (sixteen consecutive rows of one piece at a
// time, 64 banks) meet rows r and r + 8 on the same banks and take 8 cycles instead of 4 -- measured, and measured
// not to matter: the LDS pipe is a third busy in these kernels.
// The loads are inline assembly, so the compiler neither tracks them in its s_waitcnt bookkeeping nor knows that
// they write LDS: the kernels wait for them with wait_vm<N> (N = loads issued after the ones waited for; loads
// return in order, and the compiler's own counts can only wait longer than needed) and order them against their
// LDS reads with wait_lgkm0; both carry a memory clobber, so no LDS access moves across them.
// -------------------------------------------------------------------------------------------------
// An empty use of operand registers.  The compiler waits for the loads that fill them before this point -- else it
// puts that wait at their first use inside the tile loop, as vmcnt(0), where it would also wait, on every
// iteration, for the tile loads just issued (which it does not know of).
template <int N>
__device__ __forceinline__ void settle(const bf16x8 (&x)[N]) {
#pragma unroll
    for (int t = 0; t < N; ++t) asm volatile("" ::"v"(x[t]));
}
template <int D>
struct DmaTile {
    static constexpr int ROW = D * 2;     // bytes per LDS row
    static constexpr int TILE = 32 * ROW;  // 2 KB (D = 32) or 4 KB (D = 64)
    static constexpr int CPR = D / 8;      // 16-byte pieces per row
    static constexpr int NI = D / 16;      // instructions per tile, 64 / CPR rows each
    __device__ static __forceinline__ int swz(int row) {
        if constexpr (D == 64) return ((row & 3) << 1) | ((row >> 2) & 1);
        else return (((row >> 1) & 1) << 1) | ((row >> 2) & 1);
    }
    // Lane offset into the head slice (bytes): lane l fills LDS piece l of every instruction's 1 KB, i.e. position
    // l % CPR of row l / CPR (+ 64 / CPR rows per instruction), with the global piece that belongs there.
    __device__ static __forceinline__ int voff(int l, int ld) {
        const int r = l / CPR, c = (l % CPR) ^ swz(r);
        return (r * ld + c * 8) * 2;
    }
    // what the scalar offset advances by from one instruction to the next, beyond the 1024 its immediate adds
    __device__ static __forceinline__ int extra_step(int ld) { return (64 / CPR) * ld * 2 - 1024; }
    __device__ static __forceinline__ void load(u32x4 r, unsigned lds, int lvoff, int soff, int xstep) {
        if constexpr (D == 64)
            asm volatile(
                "s_mov_b32 m0, %0\n\ts_nop 3\n\t"
                "buffer_load_dwordx4 %1, %2, %3 offen lds\n\t"
                "buffer_load_dwordx4 %1, %2, %4 offen offset:1024 lds\n\t"
                "buffer_load_dwordx4 %1, %2, %5 offen offset:2048 lds\n\t"
                "buffer_load_dwordx4 %1, %2, %6 offen offset:3072 lds" ::"s"(lds),
                "v"(lvoff), "s"(r), "s"(soff), "s"(soff + xstep), "s"(soff + 2 * xstep), "s"(soff + 3 * xstep)
                : "memory");
        else
            asm volatile(
                "s_mov_b32 m0, %0\n\ts_nop 3\n\t"
                "buffer_load_dwordx4 %1, %2, %3 offen lds\n\t"
                "buffer_load_dwordx4 %1, %2, %4 offen offset:1024 lds" ::"s"(lds),
                "v"(lvoff), "s"(r), "s"(soff), "s"(soff + xstep)
                : "memory");
    }
    // Byte offsets of lane (row li, half h) for its operand over the head dimension: features h*D/2 + 8t .. of row
    // li, t = 0 .. D/16-1 (piece h*CPR/2 + t).
    struct RowAddr {
        int a[D / 16];
    };
    __device__ static __forceinline__ RowAddr row_addr(int li, int h) {
        RowAddr x;
#pragma unroll
        for (int t = 0; t < D / 16; ++t) x.a[t] = li * ROW + 16 * ((h * (CPR / 2) + t) ^ swz(li));
        return x;
    }
    __device__ static __forceinline__ void get_rows(const char* T, const RowAddr& ra, bf16x8 (&x)[D / 16]) {
#pragma unroll
        for (int t = 0; t < D / 16; ++t) x[t] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(T + ra.a[t]));
    }
    // Transposing reads (see LdsTile::get_tile_t): lane j of a group of 16 points at features F + 4(j%4) .. +3 of
    // row R + j/4, R = 4h (+ 16t, + 8), F = 16*((l/16)%2) (+ 32c): 8 bytes inside piece 2*((l/16)%2) + (j%4)/2
    // (+ 4c).  Rows 8 apart share their permutation, so the row steps stay immediate offsets.
    struct TrAddr {
        int a[D / 32];
    };
    __device__ static __forceinline__ TrAddr tr_addr(int l) {
        const int h = l >> 5, gm = (l >> 4) & 1, j = l & 15, row = 4 * h + (j >> 2);
        TrAddr x;
#pragma unroll
        for (int c = 0; c < D / 32; ++c)
            x.a[c] = row * ROW + 16 * ((4 * c + 2 * gm + ((j & 3) >> 1)) ^ swz(row)) + 8 * (j & 1);
        return x;
    }
    __device__ static __forceinline__ void get_tile_t(const char* T, const TrAddr& ta, bf16x8 (&xt)[D / 32][2]) {
        typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
#pragma unroll
        for (int c = 0; c < D / 32; ++c)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(T + ta.a[c] + (16 * t) * ROW));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(T + ta.a[c] + (16 * t + 8) * ROW));
                xt[c][t] = __builtin_shufflevector(__builtin_bit_cast(bf16x4, lo), __builtin_bit_cast(bf16x4, hi), 0, 1,
                                                   2, 3, 4, 5, 6, 7);
            }
    }
    // LDS of one wavefront: two buffers of two tiles and 256 bytes of per-tile scalars (key penalties or row
    // statistics of the tile, 64 floats)
    static constexpr int BUF = 2 * TILE + 256;
    static constexpr int WAVE = 2 * BUF;
};

// x of the lower and of the upper half-wave lane with the same lane%32, by v_permlane32_swap (exchanges the
// upper half of its first operand with the lower half of its second).  Written as inline assembly with two
// read-write operands: they must be different registers for the exchange to mean anything.
__device__ __forceinline__ void half_swap(float x, float& lo, float& hi) {
    float a = x, b = x;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    lo = a;  // {x of lanes 0-31, x of lanes 0-31}
    hi = b;  // {x of lanes 32-63, x of lanes 32-63}
}
__device__ __forceinline__ float half_swap_max(float x) {
    float lo, hi;
    half_swap(x, lo, hi);
    return fmaxf(lo, hi);
}
__device__ __forceinline__ float half_swap_sum(float x) {
    float lo, hi;
    half_swap(x, lo, hi);
    return lo + hi;
}

// The schedule of a launch (built on the host, see build_bf16_plan): every work-group is one persistent wavefront
// ("lane") that walks entries lane_ptr[b] .. lane_ptr[b+1]-1 of lane_ent, each {head, item}; an item is
// {strip, first tile, tiles, kind} with kind >= 0: chunk of a long strip whose partial result goes to workspace slot
// `kind`; -1: a whole strip; -2 (forward): strips `strip` and `strip + 1` together.
struct Bf16Sched {
    const int* items;
    const int* lane_ptr;
    const int* lane_ent;
};
#define SPION_BF16_LANE(OCC) __global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
// The index arrays never change while a kernel runs: read through the constant address space, loads with a uniform
// address are scalar loads wherever they stand (left in the global address space, the compiler turns those that
// follow a store or an assembly statement into vector loads, whose waits would also wait for the tile loads).
typedef const __attribute__((address_space(4))) int* const_ints;
__device__ __forceinline__ const_ints as_constant(const int* p) { return (const_ints) reinterpret_cast<unsigned long long>(p); }
struct LaneEntry {
    int x, y;  // head, item
};
struct PlanItem {
    int x, y, z, w;  // strip, first tile, tiles, kind
};
__device__ __forceinline__ LaneEntry lane_entry(const_ints ents, int e) { return LaneEntry{ents[2 * e], ents[2 * e + 1]}; }
__device__ __forceinline__ PlanItem plan_item(const_ints items, int k) {
    return PlanItem{items[4 * k], items[4 * k + 1], items[4 * k + 2], items[4 * k + 3]};
}
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// floats per workspace slot: two 32 x D results (the column pass has dK and dV) and 64 row statistics
template <int D>
constexpr int bf16_slot_floats() { return 2 * 32 * D + 64; }

// Byte offset of head bh inside a tensor (the tile loads address whole tensors: one resource for all heads)
template <bool ST, int D>
__device__ __forceinline__ unsigned bf16_head_bytes(const HeadLayout& y, int H, int bh, int L) {
    if constexpr (ST) {
        const int b = bh / H, hh = bh - b * H;
        return (unsigned)(((size_t)b * y.bstride + (size_t)hh * y.hstride) * 2);
    } else {
        return (unsigned)((size_t)bh * L * D * 2);
    }
}

// A 32 x D result held as acc[c][r] of lane (li, h) = row li, feature 32c + acc_row(r, h), written as bf16 rows
// through an LDS tile T: every lane writes its 8-byte pieces into the permuted tile image (DmaTile), the tile is
// read back 1 KB per instruction and stored with the lane offsets of the tile loads -- whole rows per store
// instruction where every lane storing pieces of its own row would touch 32 cache lines per instruction.
// soff: byte offset of the strip's first row.
template <int D>
__device__ __forceinline__ void stage_store_bf16(const f32x16 (&acc)[D / 32], char* T, rsrc_t r, int lvoff, int soff,
                                                 int ld, int l) {
    typedef DmaTile<D> DT;
    const int li = l & 31, h = l >> 5;
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            bf16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = (__bf16)acc[c][4 * g + e];
            *reinterpret_cast<u32x2*>(T + li * DT::ROW + 16 * ((4 * c + g) ^ DT::swz(li)) + 8 * h) = __builtin_bit_cast(u32x2, v);
        }
#pragma unroll
    for (int i = 0; i < DT::NI; ++i) {
        const u32x4 x = *reinterpret_cast<const u32x4*>(T + 1024 * i + 16 * l);
        store_b128(x, r, lvoff, soff + i * (64 / DT::CPR) * ld * 2);
    }
}
// The same result as fp32 into a workspace slot (chunk of a long strip): register (c, r) of lane l at [(16c + r)*64 + l].
template <int D>
__device__ __forceinline__ void store_part(const f32x16 (&acc)[D / 32], float* part, int l) {
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) part[(16 * c + r) * 64 + l] = acc[c][r];
}

// A lane's loads form one stream across its items.  Every element of the stream is the same three loads -- two
// 32 x D tiles into the two tile slots of an LDS buffer and 256 bytes into its third slot -- and is either a tile
// of the item (a K and a V tile and the key penalties; in the column pass a Q and a dO tile and the statistics of
// the query strip) or, ahead of the item's tiles, the strip's own operands, which reach the registers through LDS
// like everything else: loads whose lanes each fetch pieces of their own row cost the memory pipeline a cache-line
// look-up per lane, and, completing in order with the tile loads, would hold the whole stream up.
// Element number g of the stream lives in buffer g % 2; the loads of element g + 2 are issued as soon as element g
// has left its buffer -- also when it belongs to the lane's next item, so the stream does not drain at item
// boundaries.  An item's last element keeps its buffer a little longer: the item's result is staged there
// (stage_store_bf16).  The kernels keep
//   g   number of the element being worked on,   gi  elements issued so far (g <= gi <= g + 3),
//   and the kind and scalar offsets of element gi, looked up one element ahead of its issue.
// At the start of an element its loads are the oldest outstanding ones and at most one younger batch exists.
enum { EL_TILE = 0, EL_A = 1, EL_B = 2 };

// -------------------------------------------------------------------------------------------------
// Forward: one sweep per block row with a lazily raised running maximum.  PAIRS: the launch walks the pair plan,
// whose items of kind -2 give a wavefront strips 2p and 2p+1 (masks of 64 x 64 blocks and larger, where the two
// hold the same block columns): every K and V tile is fetched and read back as an operand once for the two strips'
// chains, and the two softmax updates are independent instruction streams.
// Stream of an item: {Q tile of the strip (twice, or of both strips of a pair)}, then its K / V tiles.
// -------------------------------------------------------------------------------------------------
template <int D, bool MASK, bool ST, bool PAIRS>
SPION_BF16_LANE(2) void bf16_fwd_kernel(
    const __bf16* __restrict__ Q, const __bf16* __restrict__ K, const __bf16* __restrict__ V,
    const float* __restrict__ pen, __bf16* __restrict__ O, float* __restrict__ Lse, const int* __restrict__ tcol,
    const int* __restrict__ plan_items, const int* __restrict__ lane_ptr, const int* __restrict__ lane_ent, int L,
    int NB, float scale, float* __restrict__ Part, int n_slots, Layouts ly, unsigned in_bytes, unsigned out_bytes) {
    typedef DmaTile<D> DT;
    __shared__ __attribute__((aligned(16))) char Tw[DT::WAVE];
    const int l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int e0 = as_constant(lane_ptr)[blockIdx.x], e1 = as_constant(lane_ptr)[blockIdx.x + 1];
    if (e0 >= e1) return;
    const const_ints ents = as_constant(lane_ent), items = as_constant(plan_items), tiles = as_constant(tcol);
    const int ild = ST ? ly.in.ld : D, old_ = ST ? ly.out.ld : D;
    const u32x4 wQ = rsrc_words(Q, in_bytes), wK = rsrc_words(K, in_bytes), wV = rsrc_words(V, in_bytes);
    const u32x4 wM = rsrc_words(MASK ? (const void*)pen : (const void*)K, MASK ? (size_t)NB * L * 4 : in_bytes);
    const rsrc_t rO = make_rsrc(O, out_bytes);
    const int t_bytes = 32 * ild * 2;
    const int vin = DT::voff(l, ild), xin = DT::extra_step(ild), vout = DT::voff(l, old_);
    const unsigned lds_w = lds_address(Tw);
    const typename DT::RowAddr ra = DT::row_addr(li, h);
    const typename DT::TrAddr ta = DT::tr_addr(l);
    const float c2 = scale * LOG2E, pen_mul = -1.0f / scale;
    constexpr int E = 1, OPS = 2 * DT::NI + 1;

    LaneEntry en = lane_entry(ents, e0);
    PlanItem itn = plan_item(items, en.y);
    int g = 0, gi = 0;
    int sk = 0, sa = 0, sb = 0, sc = 0, sq_g = -1;  // element sq_g: kind and the offsets of its three loads
    for (int e = e0; e < e1; ++e) {
        const int bh = en.x;
        const PlanItem it = itn;
        const bool has_next = e + 1 < e1;
        if (has_next) {
            en = lane_entry(ents, e + 1);
            itn = plan_item(items, en.y);
        }
        const int bhn = en.x;
        const int I = it.x, t0 = it.y, n = it.z;
        const bool pair = PAIRS && it.w == -2;
        const int In = itn.x, t0n = itn.y;
        const bool pairn = PAIRS && itn.w == -2;
        const int len = E + n, lenn = has_next ? E + itn.z : 0;
        const int g0 = g;
        const unsigned hb = bf16_head_bytes<ST, D>(ly.in, ly.H, bh, L), hbn = bf16_head_bytes<ST, D>(ly.in, ly.H, bhn, L);
        // element k of an item (given by value: selecting between variables captured by reference would pin them to
        // memory)
        auto locate_in = [&](int k, int bhX, int IX, int t0X, unsigned hbX, bool pairX) __attribute__((always_inline)) {
            if (k == 0) {
                sk = EL_A;
                sa = uniform((int)(hbX + (unsigned)(IX * t_bytes)));
                sb = uniform((int)(hbX + (unsigned)((IX + (pairX ? 1 : 0)) * t_bytes)));
                sc = sa;
            } else {
                const int J = tiles[t0X + k - E];
                sk = EL_TILE;
                sa = uniform((int)(hbX + (unsigned)(J * t_bytes)));
                sb = sa;
                sc = MASK ? uniform((bhX * L + J * 32) * 4) : sa;
            }
        };
        auto locate = [&, bh, bhn, I, In, t0, t0n, hb, hbn, pair, pairn, len, g0](int gg) __attribute__((always_inline)) {
            const int k = gg - g0;
            if (k < len) locate_in(k, bh, I, t0, hb, pair);
            else locate_in(k - len, bhn, In, t0n, hbn, pairn);
            sq_g = gg;
        };
        auto issue = [&]() __attribute__((always_inline)) {  // element gi -> buffer gi % 2, then look the following one up
            const unsigned a = lds_w + (gi & 1) * DT::BUF;
            if (sk == EL_TILE) {
                DT::load(wK, a, vin, sa, xin);
                DT::load(wV, a + DT::TILE, vin, sb, xin);
                dma_b32(wM, a + 2 * DT::TILE, l * 4, sc);
            } else {
                DT::load(wQ, a, vin, sa, xin);
                DT::load(wQ, a + DT::TILE, vin, sb, xin);
                dma_b32(wQ, a + 2 * DT::TILE, l * 4, sc);
            }
            ++gi;
            if (gi - g0 < len + lenn) locate(gi);
        };
        auto begin = [&]() __attribute__((always_inline)) -> char* {  // wait for element g
            if (gi - g > 1) wait_vm<OPS>();
            else wait_vm<0>();
            return Tw + (g & 1) * DT::BUF;
        };
        auto release = [&]() __attribute__((always_inline)) {  // element g has left its buffer
            wait_lgkm0();
#pragma unroll
            for (int k = 0; k < 2; ++k)
                if (gi <= g + 2 && gi - g0 < len + lenn) {
                    if (sq_g != gi) locate(gi);  // the tile loop's short cut issues without looking up
                    issue();
                }
        };
#pragma unroll
        for (int k = 0; k < 2; ++k)
            if (gi < g0 + min(2, len)) {
                if (sq_g != gi) locate(gi);
                issue();
            }
        float* part = it.w >= 0 ? Part + ((size_t)bh * n_slots + it.w) * bf16_slot_floats<D>() : nullptr;
        const unsigned ho = bf16_head_bytes<ST, D>(ly.out, ly.H, bh, L);
        // one tile: the operands leave LDS, the buffer goes to the element after next (the item's last tile keeps
        // it for the result), `math` does the arithmetic
        // Short cut for all but an item's last two tiles: the element after next is tile i + 2 of the same item, so
        // its loads need one index look-up and none of the general stream's case distinctions (which cost more
        // scalar instructions and branches per tile than the tile's arithmetic has MFMAs).
        auto tile = [&](int i, auto&& math) __attribute__((always_inline)) {
            const bool last = i + 1 == n;
            const bool quick = i + 2 < n && gi == g + 2;
            int J2 = 0;
            if (quick) J2 = tiles[t0 + i + 2];
            const char* Tk;
            if (quick) {
                wait_vm<OPS>();
                Tk = Tw + (g & 1) * DT::BUF;
            } else {
                Tk = begin();
            }
            const char* Tv = Tk + DT::TILE;
            bf16x8 kr[D / 16], vt[D / 32][2];
            DT::get_rows(Tk, ra, kr);
            DT::get_tile_t(Tv, ta, vt);
            f32x16 init = splat16(0.f);
            if constexpr (MASK) {
                float pj[16];
                lds_get_rows(reinterpret_cast<const float*>(Tk + 2 * DT::TILE), 0, h, pj);  // pj[r] = pen[acc_row(r, h)]
#pragma unroll
                for (int r = 0; r < 16; ++r) init[r] = pj[r] * pen_mul;
            }
            if (quick) {
                wait_lgkm0();
                const unsigned a = lds_w + (g & 1) * DT::BUF;  // element g + 2 takes the buffer of element g
                const int s2 = uniform((int)(hb + (unsigned)(J2 * t_bytes)));
                DT::load(wK, a, vin, s2, xin);
                DT::load(wV, a + DT::TILE, vin, s2, xin);
                dma_b32(wM, a + 2 * DT::TILE, l * 4, MASK ? uniform((bh * L + J2 * 32) * 4) : s2);
                ++gi;
            } else if (!last) {
                release();
            } else {
                wait_lgkm0();
            }
            __builtin_amdgcn_sched_barrier(0);
            math(kr, vt, init);
            __builtin_amdgcn_sched_barrier(0);
            if (!last) ++g;
        };
        // Floor of the running maximum (the reference's max(-100, .) / max(0, .), models/block_attn.cu:52): any
        // value gives the same probabilities; 2^-100 keeps (L - n) * 2^-m finite in fp32 for empty rows.
        auto update = [&](const f32x16& s, float& m, float& z, f32x16 (&o)[D / 32], bf16x8 (&pb)[2]) __attribute__((always_inline)) {
            const float t2 = half_swap_max(max16(s, -3.0e38f)) * c2;
            if (__builtin_amdgcn_ballot_w64(t2 > m + BF16_LAZY) != 0) {
                const float mn = t2 > m + BF16_LAZY ? t2 : m;
                const float f = __builtin_amdgcn_exp2f(m - mn);
                z *= f;
#pragma unroll
                for (int cc = 0; cc < D / 32; ++cc) o[cc] *= f;
                m = mn;
            }
            float p[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                p[r] = __builtin_amdgcn_exp2f(fmaf(s[r], c2, -m));
                z += p[r];
            }
            pack16(p, pb);
        };
        // rows_all: tiles of the whole strip; T: where the result is staged (a chunk finishes nothing: the merge
        // kernel does)
        auto finish = [&](float m, float z, f32x16 (&o)[D / 32], int strip, int rows_all, float* pt, char* T) __attribute__((always_inline)) {
            z = half_swap_sum(z);
            if (pt) {  // chunk of a long strip: unnormalised sums relative to m
                if (h == 0) {
                    pt[2 * 32 * D + li] = m;
                    pt[2 * 32 * D + 32 + li] = z;
                }
                store_part<D>(o, pt, l);
                return;
            }
            const int off_pattern = L - rows_all * 32;
            if (off_pattern > 0) z += (float)off_pattern * __builtin_amdgcn_exp2f(-m);  // models/block_attn.cu:74
            const float rinv = 1.0f / z;
#pragma unroll
            for (int cc = 0; cc < D / 32; ++cc) o[cc] *= rinv;
            if (h == 0) Lse[(size_t)bh * L + strip * 32 + li] = m + __builtin_amdgcn_logf(z);
            stage_store_bf16<D>(o, T, rO, vout, (int)(ho + (unsigned)(strip * 32 * old_ * 2)), old_, l);
        };
        if (pair) {
            char* Ta = begin();
            bf16x8 q0[D / 16], q1[D / 16];
            DT::get_rows(Ta, ra, q0);
            DT::get_rows(Ta + DT::TILE, ra, q1);
            if (n > 0) {
                release();
                ++g;
            }
            float m0 = MASK ? 0.f : -100.f, z0 = 0.f, m1 = m0, z1 = 0.f;
            f32x16 o0[D / 32], o1[D / 32];
#pragma unroll
            for (int c = 0; c < D / 32; ++c) {
                o0[c] = splat16(0.f);
                o1[c] = splat16(0.f);
            }
            for (int i = 0; i < n; ++i)
                tile(i, [&](const bf16x8 (&kr)[D / 16], const bf16x8 (&vt)[D / 32][2], const f32x16& init) __attribute__((always_inline)) {
                    const f32x16 s0 = mma_feat_bf16<D>(kr, q0, init);
                    const f32x16 s1 = mma_feat_bf16<D>(kr, q1, init);
                    bf16x8 pb0[2], pb1[2];
                    update(s0, m0, z0, o0, pb0);
                    update(s1, m1, z1, o1, pb1);
                    mma_tile_bf16<D>(vt, pb0, o0);
                    mma_tile_bf16<D>(vt, pb1, o1);
                });
            char* Tl = Tw + (g & 1) * DT::BUF;  // the item's last element: its buffer stages the results
            wait_lgkm0();
            finish(m0, z0, o0, I, n, nullptr, Tl);
            finish(m1, z1, o1, I + 1, n, nullptr, Tl + DT::TILE);
        } else {
            char* Ta = begin();
            bf16x8 q[D / 16];
            DT::get_rows(Ta, ra, q);
            if (n > 0) {
                release();
                ++g;
            }
            float m = MASK ? 0.f : -100.f, z = 0.f;
            f32x16 o[D / 32];
#pragma unroll
            for (int c = 0; c < D / 32; ++c) o[c] = splat16(0.f);
            for (int i = 0; i < n; ++i)
                tile(i, [&](const bf16x8 (&kr)[D / 16], const bf16x8 (&vt)[D / 32][2], const f32x16& init) __attribute__((always_inline)) {
                    const f32x16 s = mma_feat_bf16<D>(kr, q, init);  // S^T: register = key, lane = query
                    bf16x8 pb[2];
                    update(s, m, z, o, pb);
                    mma_tile_bf16<D>(vt, pb, o);  // O^T: register = feature, lane = query
                });
            char* Tl = Tw + (g & 1) * DT::BUF;
            wait_lgkm0();
            // the whole strip's tile count decides the off-pattern term; a chunk leaves that to the merge kernel
            finish(m, z, o, I, n, part, Tl);
        }
        release();
        ++g;
    }
}

// -------------------------------------------------------------------------------------------------
// Backward, row pass: g_i = dO_i . O_i, P and dP recomputed per tile, dS' = P*(dP - g), dQ += dS'.K_J;
// the 1/sqrt(d) is applied to the 32 x d result.  Stats receives {lse2, -g} of every strip (64 floats per strip:
// the 32 lse2 values, then the 32 -g values) for the column pass.
// Stream of an item: {Q tile, dO tile, lse2 of the strip}, {O tile of the strip}, then its K / V tiles.
// -------------------------------------------------------------------------------------------------
template <int D, bool MASK, bool ST>
SPION_BF16_LANE(2) void bf16_bwd_row_kernel(
    const __bf16* __restrict__ Q, const __bf16* __restrict__ K, const __bf16* __restrict__ V,
    const __bf16* __restrict__ dO, const __bf16* __restrict__ O, const float* __restrict__ Lse,
    const float* __restrict__ pen, float* __restrict__ Stats, __bf16* __restrict__ dQ, const int* __restrict__ tcol,
    const int* __restrict__ plan_items, const int* __restrict__ lane_ptr, const int* __restrict__ lane_ent, int L,
    int NB, float scale, float* __restrict__ Part, int n_slots, Layouts ly, unsigned in_bytes, unsigned out_bytes,
    unsigned grad_bytes) {
    typedef DmaTile<D> DT;
    __shared__ __attribute__((aligned(16))) char Tw[DT::WAVE];
    const int l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int e0 = as_constant(lane_ptr)[blockIdx.x], e1 = as_constant(lane_ptr)[blockIdx.x + 1];
    if (e0 >= e1) return;
    const const_ints ents = as_constant(lane_ent), items = as_constant(plan_items), tiles = as_constant(tcol);
    const int ild = ST ? ly.in.ld : D, old_ = ST ? ly.out.ld : D, gld = ST ? ly.grad.ld : D;
    const u32x4 wQ = rsrc_words(Q, in_bytes), wK = rsrc_words(K, in_bytes), wV = rsrc_words(V, in_bytes);
    const u32x4 wG = rsrc_words(dO, out_bytes), wO = rsrc_words(O, out_bytes);
    const u32x4 wL = rsrc_words(Lse, (size_t)NB * L * 4);
    const u32x4 wM = rsrc_words(MASK ? pen : Lse, (size_t)NB * L * 4);
    const rsrc_t rdQ = make_rsrc(dQ, grad_bytes);
    const int t_bytes = 32 * ild * 2, o_bytes = 32 * old_ * 2;
    const int vin = DT::voff(l, ild), xin = DT::extra_step(ild);
    const int vout = DT::voff(l, old_), xout = DT::extra_step(old_), vgr = DT::voff(l, gld);
    const unsigned lds_w = lds_address(Tw);
    const typename DT::RowAddr ra = DT::row_addr(li, h);
    const typename DT::TrAddr ta = DT::tr_addr(l);
    const float c2 = scale * LOG2E, pen_mul = -1.0f / scale;
    constexpr int E = 2, OPS = 2 * DT::NI + 1;

    LaneEntry en = lane_entry(ents, e0);
    PlanItem itn = plan_item(items, en.y);
    int g = 0, gi = 0;
    int sk = 0, sa = 0, sb = 0, sc = 0, sq_g = -1;  // element sq_g: kind and the offsets of its three loads
    for (int e = e0; e < e1; ++e) {
        const int bh = en.x;
        const PlanItem it = itn;
        const bool has_next = e + 1 < e1;
        if (has_next) {
            en = lane_entry(ents, e + 1);
            itn = plan_item(items, en.y);
        }
        const int bhn = en.x;
        const int I = it.x, t0 = it.y, n = it.z;
        const int In = itn.x, t0n = itn.y;
        const int len = E + n, lenn = has_next ? E + itn.z : 0;
        const int g0 = g;
        const unsigned hb = bf16_head_bytes<ST, D>(ly.in, ly.H, bh, L), hbn = bf16_head_bytes<ST, D>(ly.in, ly.H, bhn, L);
        const unsigned ho = bf16_head_bytes<ST, D>(ly.out, ly.H, bh, L), hon = bf16_head_bytes<ST, D>(ly.out, ly.H, bhn, L);
        auto locate_in = [&](int k, int bhX, int IX, int t0X, unsigned hbX, unsigned hoX) __attribute__((always_inline)) {
            const int lsx = (bhX * L + IX * 32) * 4;
            if (k == 0) {
                sk = EL_A;
                sa = uniform((int)(hbX + (unsigned)(IX * t_bytes)));
                sb = uniform((int)(hoX + (unsigned)(IX * o_bytes)));
                sc = uniform(lsx);
            } else if (k == 1) {
                sk = EL_B;
                sa = uniform((int)(hoX + (unsigned)(IX * o_bytes)));
                sb = sa;
                sc = uniform(lsx);
            } else {
                const int J = tiles[t0X + k - E];
                sk = EL_TILE;
                sa = uniform((int)(hbX + (unsigned)(J * t_bytes)));
                sb = sa;
                sc = uniform(MASK ? (bhX * L + J * 32) * 4 : lsx);
            }
        };
        auto locate = [&, bh, bhn, I, In, t0, t0n, hb, hbn, ho, hon, len, g0](int gg) __attribute__((always_inline)) {
            const int k = gg - g0;
            if (k < len) locate_in(k, bh, I, t0, hb, ho);
            else locate_in(k - len, bhn, In, t0n, hbn, hon);
            sq_g = gg;
        };
        auto issue = [&]() __attribute__((always_inline)) {  // element gi -> buffer gi % 2, then look the following one up
            const unsigned a = lds_w + (gi & 1) * DT::BUF;
            if (sk == EL_TILE) {
                DT::load(wK, a, vin, sa, xin);
                DT::load(wV, a + DT::TILE, vin, sb, xin);
                dma_b32(wM, a + 2 * DT::TILE, l * 4, sc);
            } else if (sk == EL_A) {
                DT::load(wQ, a, vin, sa, xin);
                DT::load(wG, a + DT::TILE, vout, sb, xout);
                dma_b32(wL, a + 2 * DT::TILE, l * 4, sc);
            } else {
                DT::load(wO, a, vout, sa, xout);
                DT::load(wO, a + DT::TILE, vout, sb, xout);
                dma_b32(wL, a + 2 * DT::TILE, l * 4, sc);
            }
            ++gi;
            if (gi - g0 < len + lenn) locate(gi);
        };
        auto begin = [&]() __attribute__((always_inline)) -> char* {  // wait for element g
            if (gi - g > 1) wait_vm<OPS>();
            else wait_vm<0>();
            return Tw + (g & 1) * DT::BUF;
        };
        auto release = [&]() __attribute__((always_inline)) {  // element g has left its buffer
            wait_lgkm0();
#pragma unroll
            for (int k = 0; k < 2; ++k)
                if (gi <= g + 2 && gi - g0 < len + lenn) {
                    if (sq_g != gi) locate(gi);  // the tile loop's short cut issues without looking up
                    issue();
                }
        };
#pragma unroll
        for (int k = 0; k < 2; ++k)
            if (gi < g0 + min(2, len)) {
                if (sq_g != gi) locate(gi);
                issue();
            }
        float* part = it.w >= 0 ? Part + ((size_t)bh * n_slots + it.w) * bf16_slot_floats<D>() : nullptr;
        // the strip's operands: Q and dO rows and lse2, then O for the row sums g = dO . O
        bf16x8 q[D / 16], go[D / 16];
        float lse, gsum = 0.f;
        {
            const char* Ta = begin();
            DT::get_rows(Ta, ra, q);
            DT::get_rows(Ta + DT::TILE, ra, go);
            lse = reinterpret_cast<const float*>(Ta + 2 * DT::TILE)[li];
            release();
            ++g;
            const char* Tb = begin();
            bf16x8 oo[D / 16];
            DT::get_rows(Tb, ra, oo);
            if (n > 0) {
                release();
                ++g;
            } else {
                wait_lgkm0();
            }
#pragma unroll
            for (int t = 0; t < D / 16; ++t)
#pragma unroll
                for (int x = 0; x < 8; ++x) gsum = fmaf((float)go[t][x], (float)oo[t][x], gsum);
            gsum = half_swap_sum(gsum);
        }
        Stats[((size_t)bh * (L / 32) + I) * 64 + l] = h ? -gsum : lse;  // every chunk of a strip writes the same values
        const f32x16 gneg = splat16(-gsum);
        f32x16 acc[D / 32];
#pragma unroll
        for (int c = 0; c < D / 32; ++c) acc[c] = splat16(0.f);
        const int ls_item = (bh * L + I * 32) * 4;
        for (int i = 0; i < n; ++i) {
            const bool last = i + 1 == n;
            // all but the item's last two tiles: the element after next is tile i + 2 of this item (see the forward)
            const bool quick = i + 2 < n && gi == g + 2;
            int J2 = 0;
            if (quick) J2 = tiles[t0 + i + 2];
            const char* Tk;
            if (quick) {
                wait_vm<OPS>();
                Tk = Tw + (g & 1) * DT::BUF;
            } else {
                Tk = begin();
            }
            const char* Tv = Tk + DT::TILE;
            bf16x8 kr[D / 16], vr[D / 16], kt[D / 32][2];
            DT::get_rows(Tk, ra, kr);
            DT::get_rows(Tv, ra, vr);
            DT::get_tile_t(Tk, ta, kt);
            f32x16 init = splat16(0.f);
            if constexpr (MASK) {
                float pj[16];
                lds_get_rows(reinterpret_cast<const float*>(Tk + 2 * DT::TILE), 0, h, pj);  // pj[r] = pen[acc_row(r, h)]
#pragma unroll
                for (int r = 0; r < 16; ++r) init[r] = pj[r] * pen_mul;
            }
            if (quick) {
                wait_lgkm0();
                const unsigned a = lds_w + (g & 1) * DT::BUF;
                const int s2 = uniform((int)(hb + (unsigned)(J2 * t_bytes)));
                DT::load(wK, a, vin, s2, xin);
                DT::load(wV, a + DT::TILE, vin, s2, xin);
                dma_b32(wM, a + 2 * DT::TILE, l * 4, uniform(MASK ? (bh * L + J2 * 32) * 4 : ls_item));
                ++gi;
            } else if (!last) {
                release();  // the tile's operands are in registers: its buffer can take the element after next
            } else {
                wait_lgkm0();  // (the item's last tile keeps it for the result)
            }
            __builtin_amdgcn_sched_barrier(0);
            const f32x16 s = mma_feat_bf16<D>(kr, q, init);
            const f32x16 dp = mma_feat_bf16<D>(vr, go, gneg);  // dO_i . v_j - g_i
            float ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = __builtin_amdgcn_exp2f(fmaf(s[r], c2, -lse)) * dp[r];
            bf16x8 dsb[2];
            pack16(ds, dsb);
            mma_tile_bf16<D>(kt, dsb, acc);  // dQ^T: register = feature, lane = query
            __builtin_amdgcn_sched_barrier(0);
            if (!last) ++g;
        }
#pragma unroll
        for (int c = 0; c < D / 32; ++c) acc[c] *= scale;
        if (part) store_part<D>(acc, part, l);
        else stage_store_bf16<D>(acc, Tw + (g & 1) * DT::BUF, rdQ, vgr,
                                 (int)(bf16_head_bytes<ST, D>(ly.grad, ly.H, bh, L) + (unsigned)(I * 32 * gld * 2)), gld, l);
        release();
        ++g;
    }
}

// -------------------------------------------------------------------------------------------------
// Backward, row pass with two strips per wavefront (masks of 64 x 64 blocks and larger, contiguous heads): the
// launch walks the pair plan, whose items of kind -2 give a wavefront strips 2p and 2p+1.  Every K and V tile is
// fetched and read back as an operand once for the two strips' chains, which run one after the other on the same
// operand registers.  Other items of the plan (chunks of long strips) are single strips and take the first half of
// the same code.
// Stream of an item: {Q tiles of the two strips, lse2 of both}, {dO tiles}, {O tiles}, then its K / V tiles.
// -------------------------------------------------------------------------------------------------
template <int D, bool MASK>
SPION_BF16_LANE(2) void bf16_bwd_row_pair_kernel(
    const __bf16* __restrict__ Q, const __bf16* __restrict__ K, const __bf16* __restrict__ V,
    const __bf16* __restrict__ dO, const __bf16* __restrict__ O, const float* __restrict__ Lse,
    const float* __restrict__ pen, float* __restrict__ Stats, __bf16* __restrict__ dQ, const int* __restrict__ tcol,
    const int* __restrict__ plan_items, const int* __restrict__ lane_ptr, const int* __restrict__ lane_ent, int L,
    int NB, float scale, float* __restrict__ Part, int n_slots, Layouts ly, unsigned in_bytes, unsigned out_bytes,
    unsigned grad_bytes) {
    constexpr bool ST = false;
    constexpr int EL_C = 3;
    typedef DmaTile<D> DT;
    __shared__ __attribute__((aligned(16))) char Tw[DT::WAVE];
    const int l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int e0 = as_constant(lane_ptr)[blockIdx.x], e1 = as_constant(lane_ptr)[blockIdx.x + 1];
    if (e0 >= e1) return;
    const const_ints ents = as_constant(lane_ent), items = as_constant(plan_items), tiles = as_constant(tcol);
    const int ild = ST ? ly.in.ld : D, old_ = ST ? ly.out.ld : D, gld = ST ? ly.grad.ld : D;
    const u32x4 wQ = rsrc_words(Q, in_bytes), wK = rsrc_words(K, in_bytes), wV = rsrc_words(V, in_bytes);
    const u32x4 wG = rsrc_words(dO, out_bytes), wO = rsrc_words(O, out_bytes);
    const u32x4 wL = rsrc_words(Lse, (size_t)NB * L * 4);
    const u32x4 wM = rsrc_words(MASK ? pen : Lse, (size_t)NB * L * 4);
    const rsrc_t rdQ = make_rsrc(dQ, grad_bytes);
    const int t_bytes = 32 * ild * 2, o_bytes = 32 * old_ * 2;
    const int vin = DT::voff(l, ild), xin = DT::extra_step(ild);
    const int vout = DT::voff(l, old_), xout = DT::extra_step(old_), vgr = DT::voff(l, gld);
    const unsigned lds_w = lds_address(Tw);
    const typename DT::RowAddr ra = DT::row_addr(li, h);
    const typename DT::TrAddr ta = DT::tr_addr(l);
    const float c2 = scale * LOG2E, pen_mul = -1.0f / scale;
    constexpr int E = 3, OPS = 2 * DT::NI + 1;

    LaneEntry en = lane_entry(ents, e0);
    PlanItem itn = plan_item(items, en.y);
    int g = 0, gi = 0;
    int sk = 0, sa = 0, sb = 0, sc = 0, sq_g = -1;  // element sq_g: kind and the offsets of its three loads
    for (int e = e0; e < e1; ++e) {
        const int bh = en.x;
        const PlanItem it = itn;
        const bool has_next = e + 1 < e1;
        if (has_next) {
            en = lane_entry(ents, e + 1);
            itn = plan_item(items, en.y);
        }
        const int bhn = en.x;
        const int I = it.x, t0 = it.y, n = it.z;
        const bool pair = it.w == -2;
        const int In = itn.x, t0n = itn.y;
        const bool pairn = itn.w == -2;
        const int len = E + n, lenn = has_next ? E + itn.z : 0;
        const int g0 = g;
        const unsigned hb = bf16_head_bytes<ST, D>(ly.in, ly.H, bh, L), hbn = bf16_head_bytes<ST, D>(ly.in, ly.H, bhn, L);
        const unsigned ho = bf16_head_bytes<ST, D>(ly.out, ly.H, bh, L), hon = bf16_head_bytes<ST, D>(ly.out, ly.H, bhn, L);
        auto locate_in = [&](int k, int bhX, int IX, int t0X, unsigned hbX, unsigned hoX, bool pairX) __attribute__((always_inline)) {
            const int lsx = (bhX * L + IX * 32) * 4;
            const int Ib = IX + (pairX ? 1 : 0);
            if (k < E) {
                sk = k == 0 ? EL_A : k == 1 ? EL_B : EL_C;
                const unsigned base = k == 0 ? hbX : hoX;
                const int step = k == 0 ? t_bytes : o_bytes;
                sa = uniform((int)(base + (unsigned)(IX * step)));
                sb = uniform((int)(base + (unsigned)(Ib * step)));
                sc = uniform(lsx);
            } else {
                const int J = tiles[t0X + k - E];
                sk = EL_TILE;
                sa = uniform((int)(hbX + (unsigned)(J * t_bytes)));
                sb = sa;
                sc = uniform(MASK ? (bhX * L + J * 32) * 4 : lsx);
            }
        };
        auto locate = [&, bh, bhn, I, In, t0, t0n, hb, hbn, ho, hon, len, g0, pair, pairn](int gg) __attribute__((always_inline)) {
            const int k = gg - g0;
            if (k < len) locate_in(k, bh, I, t0, hb, ho, pair);
            else locate_in(k - len, bhn, In, t0n, hbn, hon, pairn);
            sq_g = gg;
        };
        auto issue = [&]() __attribute__((always_inline)) {  // element gi -> buffer gi % 2, then look the following one up
            const unsigned a = lds_w + (gi & 1) * DT::BUF;
            if (sk == EL_TILE) {
                DT::load(wK, a, vin, sa, xin);
                DT::load(wV, a + DT::TILE, vin, sb, xin);
                dma_b32(wM, a + 2 * DT::TILE, l * 4, sc);
            } else if (sk == EL_A) {
                DT::load(wQ, a, vin, sa, xin);
                DT::load(wQ, a + DT::TILE, vin, sb, xin);
                dma_b32(wL, a + 2 * DT::TILE, l * 4, sc);
            } else if (sk == EL_B) {
                DT::load(wG, a, vout, sa, xout);
                DT::load(wG, a + DT::TILE, vout, sb, xout);
                dma_b32(wL, a + 2 * DT::TILE, l * 4, sc);
            } else {
                DT::load(wO, a, vout, sa, xout);
                DT::load(wO, a + DT::TILE, vout, sb, xout);
                dma_b32(wL, a + 2 * DT::TILE, l * 4, sc);
            }
            ++gi;
            if (gi - g0 < len + lenn) locate(gi);
        };
        auto begin = [&]() __attribute__((always_inline)) -> char* {  // wait for element g
            if (gi - g > 1) wait_vm<OPS>();
            else wait_vm<0>();
            return Tw + (g & 1) * DT::BUF;
        };
        auto release = [&]() __attribute__((always_inline)) {  // element g has left its buffer
            wait_lgkm0();
#pragma unroll
            for (int k = 0; k < 2; ++k)
                if (gi <= g + 2 && gi - g0 < len + lenn) {
                    if (sq_g != gi) locate(gi);  // the tile loop's short cut issues without looking up
                    issue();
                }
        };
#pragma unroll
        for (int k = 0; k < 2; ++k)
            if (gi < g0 + min(2, len)) {
                if (sq_g != gi) locate(gi);
                issue();
            }
        float* part = it.w >= 0 ? Part + ((size_t)bh * n_slots + it.w) * bf16_slot_floats<D>() : nullptr;
        // the strips' operands: Q rows and lse2, dO rows, then O for the row sums g = dO . O
        bf16x8 qa[D / 16], qb[D / 16], ga[D / 16], gb[D / 16];
        float lse_a, lse_b, gsum_a = 0.f, gsum_b = 0.f;
        {
            const char* Ta = begin();
            DT::get_rows(Ta, ra, qa);
            DT::get_rows(Ta + DT::TILE, ra, qb);
            lse_a = reinterpret_cast<const float*>(Ta + 2 * DT::TILE)[li];
            lse_b = reinterpret_cast<const float*>(Ta + 2 * DT::TILE)[32 + li];
            release();
            ++g;
            const char* Tb = begin();
            DT::get_rows(Tb, ra, ga);
            DT::get_rows(Tb + DT::TILE, ra, gb);
            release();
            ++g;
            const char* Tc = begin();
            bf16x8 oa[D / 16], ob[D / 16];
            DT::get_rows(Tc, ra, oa);
            DT::get_rows(Tc + DT::TILE, ra, ob);
            if (n > 0) {
                release();
                ++g;
            } else {
                wait_lgkm0();
            }
#pragma unroll
            for (int t = 0; t < D / 16; ++t)
#pragma unroll
                for (int x = 0; x < 8; ++x) {
                    gsum_a = fmaf((float)ga[t][x], (float)oa[t][x], gsum_a);
                    gsum_b = fmaf((float)gb[t][x], (float)ob[t][x], gsum_b);
                }
            gsum_a = half_swap_sum(gsum_a);
            gsum_b = half_swap_sum(gsum_b);
        }
        // every chunk of a strip writes the same values
        Stats[((size_t)bh * (L / 32) + I) * 64 + l] = h ? -gsum_a : lse_a;
        if (pair) Stats[((size_t)bh * (L / 32) + I + 1) * 64 + l] = h ? -gsum_b : lse_b;
        const f32x16 gneg_a = splat16(-gsum_a), gneg_b = splat16(-gsum_b);
        f32x16 acc_a[D / 32], acc_b[D / 32];
#pragma unroll
        for (int c = 0; c < D / 32; ++c) {
            acc_a[c] = splat16(0.f);
            acc_b[c] = splat16(0.f);
        }
        const int ls_item = (bh * L + I * 32) * 4;
        for (int i = 0; i < n; ++i) {
            const bool last = i + 1 == n;
            // all but the item's last two tiles: the element after next is tile i + 2 of this item (see the forward)
            const bool quick = i + 2 < n && gi == g + 2;
            int J2 = 0;
            if (quick) J2 = tiles[t0 + i + 2];
            const char* Tk;
            if (quick) {
                wait_vm<OPS>();
                Tk = Tw + (g & 1) * DT::BUF;
            } else {
                Tk = begin();
            }
            const char* Tv = Tk + DT::TILE;
            bf16x8 kr[D / 16], vr[D / 16], kt[D / 32][2];
            DT::get_rows(Tk, ra, kr);
            DT::get_rows(Tv, ra, vr);
            DT::get_tile_t(Tk, ta, kt);
            f32x16 init = splat16(0.f);
            if constexpr (MASK) {
                float pj[16];
                lds_get_rows(reinterpret_cast<const float*>(Tk + 2 * DT::TILE), 0, h, pj);  // pj[r] = pen[acc_row(r, h)]
#pragma unroll
                for (int r = 0; r < 16; ++r) init[r] = pj[r] * pen_mul;
            }
            if (quick) {
                wait_lgkm0();
                const unsigned a = lds_w + (g & 1) * DT::BUF;
                const int s2 = uniform((int)(hb + (unsigned)(J2 * t_bytes)));
                DT::load(wK, a, vin, s2, xin);
                DT::load(wV, a + DT::TILE, vin, s2, xin);
                dma_b32(wM, a + 2 * DT::TILE, l * 4, uniform(MASK ? (bh * L + J2 * 32) * 4 : ls_item));
                ++gi;
            } else if (!last) {
                release();  // the tile's operands are in registers: its buffer can take the element after next
            } else {
                wait_lgkm0();  // (the item's last tile keeps it for the result)
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                const f32x16 s = mma_feat_bf16<D>(kr, qa, init);
                const f32x16 dp = mma_feat_bf16<D>(vr, ga, gneg_a);  // dO_i . v_j - g_i
                float ds[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) ds[r] = __builtin_amdgcn_exp2f(fmaf(s[r], c2, -lse_a)) * dp[r];
                bf16x8 dsb[2];
                pack16(ds, dsb);
                mma_tile_bf16<D>(kt, dsb, acc_a);  // dQ^T: register = feature, lane = query
            }
            if (pair) {
                const f32x16 s = mma_feat_bf16<D>(kr, qb, init);
                const f32x16 dp = mma_feat_bf16<D>(vr, gb, gneg_b);
                float ds[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) ds[r] = __builtin_amdgcn_exp2f(fmaf(s[r], c2, -lse_b)) * dp[r];
                bf16x8 dsb[2];
                pack16(ds, dsb);
                mma_tile_bf16<D>(kt, dsb, acc_b);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (!last) ++g;
        }
#pragma unroll
        for (int c = 0; c < D / 32; ++c) {
            acc_a[c] *= scale;
            acc_b[c] *= scale;
        }
        if (part) {
            store_part<D>(acc_a, part, l);
        } else {
            char* Tl = Tw + (g & 1) * DT::BUF;
            const int so = (int)(bf16_head_bytes<ST, D>(ly.grad, ly.H, bh, L) + (unsigned)(I * 32 * gld * 2));
            stage_store_bf16<D>(acc_a, Tl, rdQ, vgr, so, gld, l);
            if (pair) stage_store_bf16<D>(acc_b, Tl + DT::TILE, rdQ, vgr, so + 32 * gld * 2, gld, l);
        }
        release();
        ++g;
    }
}

// -------------------------------------------------------------------------------------------------
// Backward, column pass over the transposed tile index: dK_J = sum_I dS_IJ^T Q_I, dV_J = sum_I P_IJ^T dO_I.
// Stats: {lse2, -g} of every strip as the row pass left them (64 floats per strip).
// Stream of an item: {K tile, V tile, key penalties of the column strip}, then per tile {Q tile, dO tile, statistics
// of the query strip}.
// -------------------------------------------------------------------------------------------------
template <int D, bool MASK, bool ST>
SPION_BF16_LANE(2) void bf16_bwd_col_kernel(
    const __bf16* __restrict__ Q, const __bf16* __restrict__ K, const __bf16* __restrict__ V,
    const __bf16* __restrict__ dO, const float* __restrict__ Stats, const float* __restrict__ pen,
    __bf16* __restrict__ dK, __bf16* __restrict__ dV, const int* __restrict__ tcdesc,
    const int* __restrict__ plan_items, const int* __restrict__ lane_ptr, const int* __restrict__ lane_ent, int L, int NB,
    float scale, float* __restrict__ Part, int n_slots, Layouts ly, unsigned in_bytes, unsigned out_bytes,
    unsigned grad_bytes) {
    typedef DmaTile<D> DT;
    __shared__ __attribute__((aligned(16))) char Tw[DT::WAVE];
    const int l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int e0 = as_constant(lane_ptr)[blockIdx.x], e1 = as_constant(lane_ptr)[blockIdx.x + 1];
    if (e0 >= e1) return;
    const const_ints ents = as_constant(lane_ent), items = as_constant(plan_items);
    const const_ints tiles = as_constant(tcdesc);  // four ints per tile of the transposed index, the first its block row
    const int ild = ST ? ly.in.ld : D, old_ = ST ? ly.out.ld : D, gld = ST ? ly.grad.ld : D;
    const u32x4 wQ = rsrc_words(Q, in_bytes), wK = rsrc_words(K, in_bytes), wV = rsrc_words(V, in_bytes);
    const u32x4 wG = rsrc_words(dO, out_bytes);
    const u32x4 wS = rsrc_words(Stats, (size_t)NB * L * 8);
    const u32x4 wM = rsrc_words(MASK ? pen : Stats, (size_t)NB * L * 4);
    const rsrc_t rdK = make_rsrc(dK, grad_bytes), rdV = make_rsrc(dV, grad_bytes);
    const int t_bytes = 32 * ild * 2, o_bytes = 32 * old_ * 2;
    const int vin = DT::voff(l, ild), xin = DT::extra_step(ild);
    const int vout = DT::voff(l, old_), xout = DT::extra_step(old_), vgr = DT::voff(l, gld);
    const unsigned lds_w = lds_address(Tw);
    const typename DT::RowAddr ra = DT::row_addr(li, h);
    const typename DT::TrAddr ta = DT::tr_addr(l);
    const float c2 = scale * LOG2E;
    constexpr int E = 1, OPS = 2 * DT::NI + 1;
    // d = 64 has no registers for the transposed tiles while the first chains' operands are live: they are read
    // once the chains are issued, and the buffer is handed on after that.
    constexpr bool DEEP = D == 32;

    LaneEntry en = lane_entry(ents, e0);
    PlanItem itn = plan_item(items, en.y);
    int g = 0, gi = 0;
    int sk = 0, sa = 0, sb = 0, sc = 0, sq_g = -1;  // element sq_g: kind and the offsets of its three loads
    for (int e = e0; e < e1; ++e) {
        const int bh = en.x;
        const PlanItem it = itn;
        const bool has_next = e + 1 < e1;
        if (has_next) {
            en = lane_entry(ents, e + 1);
            itn = plan_item(items, en.y);
        }
        const int bhn = en.x;
        const int J = it.x, t0 = it.y, n = it.z;
        const int Jn = itn.x, t0n = itn.y;
        const int len = E + n, lenn = has_next ? E + itn.z : 0;
        const int g0 = g;
        const unsigned hb = bf16_head_bytes<ST, D>(ly.in, ly.H, bh, L), hbn = bf16_head_bytes<ST, D>(ly.in, ly.H, bhn, L);
        const unsigned ho = bf16_head_bytes<ST, D>(ly.out, ly.H, bh, L), hon = bf16_head_bytes<ST, D>(ly.out, ly.H, bhn, L);
        auto locate_in = [&](int k, int bhX, int JX, int t0X, unsigned hbX, unsigned hoX) __attribute__((always_inline)) {
            if (k == 0) {
                sk = EL_A;
                sa = uniform((int)(hbX + (unsigned)(JX * t_bytes)));
                sb = sa;
                sc = uniform((bhX * L + JX * 32) * 4);
            } else {
                const int I = tiles[4 * (t0X + k - E)];
                sk = EL_TILE;
                sa = uniform((int)(hbX + (unsigned)(I * t_bytes)));
                sb = uniform((int)(hoX + (unsigned)(I * o_bytes)));
                sc = uniform((bhX * (L / 32) + I) * 256);
            }
        };
        auto locate = [&, bh, bhn, J, Jn, t0, t0n, hb, hbn, ho, hon, len, g0](int gg) __attribute__((always_inline)) {
            const int k = gg - g0;
            if (k < len) locate_in(k, bh, J, t0, hb, ho);
            else locate_in(k - len, bhn, Jn, t0n, hbn, hon);
            sq_g = gg;
        };
        auto issue = [&]() __attribute__((always_inline)) {  // element gi -> buffer gi % 2, then look the following one up
            const unsigned a = lds_w + (gi & 1) * DT::BUF;
            if (sk == EL_TILE) {
                DT::load(wQ, a, vin, sa, xin);
                DT::load(wG, a + DT::TILE, vout, sb, xout);
                dma_b32(wS, a + 2 * DT::TILE, l * 4, sc);
            } else {
                DT::load(wK, a, vin, sa, xin);
                DT::load(wV, a + DT::TILE, vin, sb, xin);
                dma_b32(wM, a + 2 * DT::TILE, l * 4, sc);
            }
            ++gi;
            if (gi - g0 < len + lenn) locate(gi);
        };
        auto begin = [&]() __attribute__((always_inline)) -> char* {  // wait for element g
            if (gi - g > 1) wait_vm<OPS>();
            else wait_vm<0>();
            return Tw + (g & 1) * DT::BUF;
        };
        auto release = [&]() __attribute__((always_inline)) {  // element g has left its buffer
            wait_lgkm0();
#pragma unroll
            for (int k = 0; k < 2; ++k)
                if (gi <= g + 2 && gi - g0 < len + lenn) {
                    if (sq_g != gi) locate(gi);  // the tile loop's short cut issues without looking up
                    issue();
                }
        };
#pragma unroll
        for (int k = 0; k < 2; ++k)
            if (gi < g0 + min(2, len)) {
                if (sq_g != gi) locate(gi);
                issue();
            }
        float* part = it.w >= 0 ? Part + ((size_t)bh * n_slots + it.w) * bf16_slot_floats<D>() : nullptr;
        // the column strip's operands: K and V rows (and the key penalties)
        bf16x8 k[D / 16], v[D / 16];
        f32x16 sinit = splat16(0.f);
        {
            const char* Ta = begin();
            DT::get_rows(Ta, ra, k);
            DT::get_rows(Ta + DT::TILE, ra, v);
            if constexpr (MASK) sinit = splat16(-reinterpret_cast<const float*>(Ta + 2 * DT::TILE)[li] / scale);
            if (n > 0) {
                release();
                ++g;
            } else {
                wait_lgkm0();
            }
        }
        f32x16 ak[D / 32], av[D / 32];
#pragma unroll
        for (int c = 0; c < D / 32; ++c) {
            ak[c] = splat16(0.f);
            av[c] = splat16(0.f);
        }
        // all but the item's last two tiles: the element after next is tile i + 2 of this item (see the forward)
        auto quick_issue = [&](int I2) __attribute__((always_inline)) {
            const unsigned a = lds_w + (g & 1) * DT::BUF;
            DT::load(wQ, a, vin, uniform((int)(hb + (unsigned)(I2 * t_bytes))), xin);
            DT::load(wG, a + DT::TILE, vout, uniform((int)(ho + (unsigned)(I2 * o_bytes))), xout);
            dma_b32(wS, a + 2 * DT::TILE, l * 4, uniform((bh * (L / 32) + I2) * 256));
            ++gi;
        };
        for (int i = 0; i < n; ++i) {
            const bool last = i + 1 == n;
            const bool quick = i + 2 < n && gi == g + 2;
            int I2 = 0;
            if (quick) I2 = tiles[4 * (t0 + i + 2)];
            const char* Tq;
            if (quick) {
                wait_vm<OPS>();
                Tq = Tw + (g & 1) * DT::BUF;
            } else {
                Tq = begin();
            }
            const char* Tg = Tq + DT::TILE;
            const float* St = reinterpret_cast<const float*>(Tq + 2 * DT::TILE);  // lse2[32], -g[32] of the tile's queries
            float lse[16], gn[16];
            lds_get_rows(St, 0, h, lse);      // lse[r] = St[acc_row(r, h)]
            lds_get_rows(St + 32, 0, h, gn);  // gn[r]  = St[32 + acc_row(r, h)]
            bf16x8 qr[D / 16], gr[D / 16], qt[D / 32][2], gt[D / 32][2];
            DT::get_rows(Tq, ra, qr);
            DT::get_rows(Tg, ra, gr);
            if constexpr (DEEP) {
                DT::get_tile_t(Tq, ta, qt);
                DT::get_tile_t(Tg, ta, gt);
                if (quick) {
                    wait_lgkm0();
                    quick_issue(I2);
                } else if (!last) {
                    release();
                } else {
                    wait_lgkm0();
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            const f32x16 s = mma_feat_bf16<D>(qr, k, sinit);  // S: register = query, lane = key
            f32x16 ginit;
#pragma unroll
            for (int r = 0; r < 16; ++r) ginit[r] = gn[r];
            const f32x16 dp = mma_feat_bf16<D>(gr, v, ginit);  // dO_i . v_j - g_i
            if constexpr (!DEEP) {
                DT::get_tile_t(Tq, ta, qt);
                DT::get_tile_t(Tg, ta, gt);
            }
            float p[16], ds[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                p[r] = __builtin_amdgcn_exp2f(fmaf(s[r], c2, -lse[r]));
                ds[r] = p[r] * dp[r];
            }
            bf16x8 pb[2], dsb[2];
            pack16(p, pb);
            pack16(ds, dsb);
            if constexpr (!DEEP) {
                if (quick) {
                    wait_lgkm0();
                    quick_issue(I2);
                } else if (!last) {
                    release();
                } else {
                    wait_lgkm0();
                }
            }
            mma_tile_bf16<D>(qt, dsb, ak);  // dK^T: register = feature, lane = key
            mma_tile_bf16<D>(gt, pb, av);   // dV^T
            __builtin_amdgcn_sched_barrier(0);
            if (!last) ++g;
        }
#pragma unroll
        for (int c = 0; c < D / 32; ++c) ak[c] *= scale;
        if (part) {
            store_part<D>(ak, part, l);
            store_part<D>(av, part + 32 * D, l);
        } else {
            char* Tl = Tw + (g & 1) * DT::BUF;
            const int so = (int)(bf16_head_bytes<ST, D>(ly.grad, ly.H, bh, L) + (unsigned)(J * 32 * gld * 2));
            stage_store_bf16<D>(ak, Tl, rdK, vgr, so, gld, l);
            stage_store_bf16<D>(av, Tl + DT::TILE, rdV, vgr, so, gld, l);
        }
        release();
        ++g;
    }
}

// -------------------------------------------------------------------------------------------------
// Merge of the chunks of long strips.  desc[k] = {strip, first slot, number of chunks, tiles of the strip};
// one work-group per (head, long strip, 256 elements of the 32 x D result), one element per thread, the loads of
// up to eight chunks in flight at a time.  Element e of a slot is register (c, r) = (e / 1024, e / 64 % 16) of lane
// l = e % 64: row l % 32 of the strip, feature 32c + acc_row(r, l / 32).
// -------------------------------------------------------------------------------------------------
template <int D, bool ST>
__global__ __launch_bounds__(256) void bf16_merge_fwd_kernel(const float* __restrict__ Part, const int* __restrict__ desc,
                                                             int n_long, int n_slots, __bf16* __restrict__ O,
                                                             float* __restrict__ Lse, int L, HeadLayout lay, int H) {
    constexpr int PSZ = bf16_slot_floats<D>(), EB = 32 * D / 256;
    const int eb = blockIdx.x % EB, item = blockIdx.x / EB;
    const int bh = item / n_long;
    const int4 d = reinterpret_cast<const int4*>(desc)[item % n_long];
    const float* p0 = Part + ((size_t)bh * n_slots + d.y) * PSZ;
    const float* st = p0 + 2 * 32 * D;  // {m[32], z[32]} of chunk 0
    __shared__ float sm[32], sr[32];
    const int t = threadIdx.x;
    if (t < 32) {
        float M = -3.0e38f;
        for (int c0 = 0; c0 < d.z; c0 += 8) {
            float mm[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) mm[k] = st[(size_t)min(c0 + k, d.z - 1) * PSZ + t];
#pragma unroll
            for (int k = 0; k < 8; ++k) M = fmaxf(M, mm[k]);
        }
        float Z = 0.f;
        for (int c0 = 0; c0 < d.z; c0 += 8) {
            float mm[8], zz[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                mm[k] = st[(size_t)min(c0 + k, d.z - 1) * PSZ + t];
                zz[k] = st[(size_t)min(c0 + k, d.z - 1) * PSZ + 32 + t];
            }
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (c0 + k < d.z) Z += zz[k] * __builtin_amdgcn_exp2f(mm[k] - M);
        }
        const int off_pattern = L - d.w * 32;
        if (off_pattern > 0) Z += (float)off_pattern * __builtin_amdgcn_exp2f(-M);  // models/block_attn.cu:74
        sm[t] = M;
        sr[t] = 1.0f / Z;
        if (eb == 0) Lse[(size_t)bh * L + d.x * 32 + t] = M + __builtin_amdgcn_logf(Z);
    }
    __syncthreads();
    const int e = eb * 256 + t;
    const int l = e & 63, r = (e >> 6) & 15, c = e >> 10, row = l & 31;
    float v = 0.f;
    for (int c0 = 0; c0 < d.z; c0 += 8) {
        float x[8], mm[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            x[k] = p0[(size_t)min(c0 + k, d.z - 1) * PSZ + e];
            mm[k] = st[(size_t)min(c0 + k, d.z - 1) * PSZ + row];
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (c0 + k < d.z) v += x[k] * __builtin_amdgcn_exp2f(mm[k] - sm[row]);
    }
    size_t ob, obytes;
    int old_;
    bf16_head<ST, D>(lay, H, bh, L, ob, old_, obytes);
    O[ob + (size_t)(d.x * 32 + row) * old_ + 32 * c + acc_row(r, l >> 5)] = (__bf16)(v * sr[row]);
}

// Plain sums (backward): out0 from the first 32 x D block of the slots, out1 (column pass: dV; grid twice as
// large) from the second.
template <int D, bool ST>
__global__ __launch_bounds__(256) void bf16_merge_sum_kernel(const float* __restrict__ Part, const int* __restrict__ desc,
                                                             int n_long, int n_slots, __bf16* __restrict__ out0,
                                                             __bf16* __restrict__ out1, int L, HeadLayout lay, int H) {
    constexpr int PSZ = bf16_slot_floats<D>();
    const int EB = (out1 ? 2 : 1) * 32 * D / 256;
    const int eb = blockIdx.x % EB, item = blockIdx.x / EB;
    const int bh = item / n_long;
    const int4 d = reinterpret_cast<const int4*>(desc)[item % n_long];
    const float* p0 = Part + ((size_t)bh * n_slots + d.y) * PSZ;
    const int e = eb * 256 + threadIdx.x;
    const int which = e / (32 * D), ee = e % (32 * D);
    const int l = ee & 63, r = (ee >> 6) & 15, c = ee >> 10, row = l & 31;
    float v = 0.f;
    for (int c0 = 0; c0 < d.z; c0 += 8) {
        float x[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) x[k] = p0[(size_t)min(c0 + k, d.z - 1) * PSZ + e];
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (c0 + k < d.z) v += x[k];
    }
    size_t gb, gbytes;
    int gld;
    bf16_head<ST, D>(lay, H, bh, L, gb, gld, gbytes);
    (which ? out1 : out0)[gb + (size_t)(d.x * 32 + row) * gld + 32 * c + acc_row(r, l >> 5)] = (__bf16)v;
}

}  // namespace spion
