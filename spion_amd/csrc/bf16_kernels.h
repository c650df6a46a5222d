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
// Tiles travel global memory -> registers (consecutive addresses across the wavefront, one tile ahead) ->
// wave-private LDS tile -> operand layouts; same-wave LDS accesses complete in order, so no barrier is involved.
// Queries are the lane index of every row-pass accumulator (S^T, dP^T, O^T, dQ^T), so row statistics are
// lane scalars; keys are the lane index in the column pass.
//
// Work-groups have four wavefronts and take one entry of a host-built list: four short strips (one per
// wavefront, no barriers) or one chunk of a long strip (a global row or column) walked by the four wavefronts
// together.  A long strip is cut into chunks of about the work of an ordinary work-group, so that it does not
// outlast the rest of the launch; every chunk leaves fp32 partial results in a workspace slot and a small
// merge kernel combines the slots of a strip.
#pragma once
#include "tile_kernels.h"

namespace spion {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

constexpr int BF16_WAVES = 4;
// OCC wavefronts per SIMD: what the registers of each variant allow without spilling (measured: going from two to
// three or four changes little, the kernels are bound by the instruction mix of a tile, not by latency).
#define SPION_BF16_KERNEL(OCC) \
    __global__ __launch_bounds__(64 * BF16_WAVES) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
constexpr float BF16_LAZY = 8.f;  // the running row maximum is raised only when a tile exceeds it by 2^8

template <int D>
__device__ __forceinline__ void ldb_rows(rsrc_t r, int voff, int soff, bf16x8 (&x)[D / 16]) {
#pragma unroll
    for (int t = 0; t < D / 16; ++t)
        x[t] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff + 16 * t, 0));
}

// A 32 x D bf16 tile of a row-major head slice is 64*D consecutive bytes.  Loaded as D/16 instructions in which
// the 64 lanes read 1 KB of consecutive addresses: 8 cache lines per instruction.  (Reading it directly in the
// operand layout -- every lane 16 bytes of its own row -- costs one tag lookup per lane and was measured to
// keep the texture path busy 84 % of the time.)  Lane l, instruction i holds 16-byte piece 64i + l of the tile.
// With rows ld elements apart (a head that is a view of a wider buffer) the same pieces come from 512 / D rows per
// instruction: lane offset bf16_tile_voff, `step` = bf16_tile_step bytes from one instruction to the next.
template <int D>
__device__ __forceinline__ void ldb_tile(rsrc_t r, int lvoff, int soff, int step, u32x4 (&raw)[D / 16]) {
#pragma unroll
    for (int i = 0; i < D / 16; ++i) raw[i] = __builtin_amdgcn_raw_buffer_load_b128(r, lvoff, soff + step * i, 0);
}
template <int D>
__device__ __forceinline__ int bf16_tile_voff(int l, int ld) {
    constexpr int PPR = D / 8;  // 16-byte pieces per row
    return ((l / PPR) * ld + (l % PPR) * 8) * 2;
}
template <int D>
__device__ __forceinline__ int bf16_tile_step(int ld) {
    return (512 / D) * ld * 2;
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

// Wave-private LDS tile of 32 row-major rows of D bf16, rows RS bytes apart.
template <int D>
struct LdsTile {
    static constexpr int RS = D * 2 + 32;
    static constexpr int BYTES = 32 * RS;
    // lane (row li, half h) stores the D/2 features it holds as a head-dimension operand
    static __device__ __forceinline__ void put_rows(char* T, int li, int h, const bf16x8 (&x)[D / 16]) {
#pragma unroll
        for (int t = 0; t < D / 16; ++t) *reinterpret_cast<u32x4*>(T + li * RS + h * D + 16 * t) = __builtin_bit_cast(u32x4, x[t]);
    }
    // the tile as loaded by ldb_tile: piece 64i + l is row (64i + l) / (D/8), 16-byte column (64i + l) % (D/8)
    static __device__ __forceinline__ void put_raw(char* T, int l, const u32x4 (&raw)[D / 16]) {
        constexpr int CPR = D / 8;
#pragma unroll
        for (int i = 0; i < D / 16; ++i)
            *reinterpret_cast<u32x4*>(T + ((64 * i) / CPR + l / CPR) * RS + (l % CPR) * 16) = raw[i];
    }
    // head-dimension operand of lane (row li, half h): features h*D/2 ..
    static __device__ __forceinline__ void get_rows(const char* T, int li, int h, bf16x8 (&x)[D / 16]) {
#pragma unroll
        for (int t = 0; t < D / 16; ++t)
            x[t] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(T + li * RS + h * D + 16 * t));
    }
    // The transposing read works on groups of 16 lanes: lane j of a group points at 4 consecutive bf16,
    // and lane 4a+b receives element b of the pieces of lanes a, 4+a, 8+a, 12+a.  With lane j pointing at
    // row R + j/4, features F + 4(j%4) .., lane 4a+b gets rows R..R+3 of feature F + 4a + b.
    // lane_base: byte offset of this lane's piece for R = 4h, F = 16*((l/16)%2).
    static __device__ __forceinline__ int lane_base(int l) {
        const int h = l >> 5, gm = (l >> 4) & 1, j = l & 15;
        return (4 * h + (j >> 2)) * RS + (16 * gm + 4 * (j & 3)) * 2;
    }
    static __device__ __forceinline__ void get_tile_t(const char* T, int base, bf16x8 (&xt)[D / 32][2]) {
        typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
#pragma unroll
        for (int c = 0; c < D / 32; ++c)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(T + base + (16 * t) * RS + c * 64));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(T + base + (16 * t + 8) * RS + c * 64));
                xt[c][t] = __builtin_shufflevector(__builtin_bit_cast(bf16x4, lo), __builtin_bit_cast(bf16x4, hi), 0, 1,
                                                   2, 3, 4, 5, 6, 7);
            }
    }
};

// -------------------------------------------------------------------------------------------------
// Tiles that go from global memory straight into LDS (buffer loads with the LDS modifier): no registers hold a
// tile in flight and no ds_write is spent on it.  One instruction moves 64 x 16 bytes to 1 KB of consecutive LDS
// addresses starting at M0 (+ the instruction's immediate offset, which is added to the global address as well);
// which 16-byte piece of global memory a lane fetches is free, so the LDS image of a tile is unpadded rows with
// the pieces of a row permuted: piece c of tile row r lies at position c ^ swz(r).  With that permutation both
// kinds of LDS reads are free of bank conflicts: eight consecutive rows of one piece (operand over the head
// dimension, ds_read_b128) and four consecutive rows of two adjacent pieces (transposing read).
// The loads are inline assembly, so the compiler neither tracks them in its s_waitcnt bookkeeping nor knows that
// they write LDS: the kernels wait for them with wait_vm<N> (N = loads issued after the ones waited for; loads
// return in order, and the compiler's own counts can only wait longer than needed) and order them against their
// LDS reads with wait_lgkm0; both carry a memory clobber, so no LDS access moves across them.
// -------------------------------------------------------------------------------------------------
__device__ __forceinline__ u32x4 rsrc_words(const void* p, size_t bytes) {
    const unsigned long long a = reinterpret_cast<unsigned long long>(p);
    u32x4 r;
    r.x = (unsigned)a;
    r.y = (unsigned)(a >> 32);  // stride 0, no swizzle
    r.z = bytes > 0xfffffff0ull ? 0xfffffff0u : (unsigned)bytes;
    r.w = 0x00020000u;
    // wave-uniform by construction; keep it in scalar registers
    r.x = __builtin_amdgcn_readfirstlane(r.x);
    r.y = __builtin_amdgcn_readfirstlane(r.y);
    r.z = __builtin_amdgcn_readfirstlane(r.z);
    return r;
}
__device__ __forceinline__ unsigned lds_address(const void* p) {
    typedef __attribute__((address_space(3))) const char* lds_ptr;
    return __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<unsigned long long>((lds_ptr)p));
}
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// An empty use of operand registers.  The compiler waits for the loads that fill them before this point -- else it
// puts that wait at their first use inside the tile loop, as vmcnt(0), where it would also wait, on every
// iteration, for the tile loads just issued (which it does not know of).
template <int N>
__device__ __forceinline__ void settle(const bf16x8 (&x)[N]) {
#pragma unroll
    for (int t = 0; t < N; ++t) asm volatile("" ::"v"(x[t]));
}
__device__ __forceinline__ void settle(float x) { asm volatile("" ::"v"(x)); }
// 64 floats (lane l: 4 bytes at voff) to 256 bytes of LDS
__device__ __forceinline__ void dma_b32(u32x4 r, unsigned lds, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds" ::"s"(lds), "v"(voff), "s"(r),
                 "s"(soff)
                 : "memory");
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
                "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                "buffer_load_dwordx4 %1, %2, %3 offen lds\n\t"
                "buffer_load_dwordx4 %1, %2, %4 offen offset:1024 lds\n\t"
                "buffer_load_dwordx4 %1, %2, %5 offen offset:2048 lds\n\t"
                "buffer_load_dwordx4 %1, %2, %6 offen offset:3072 lds" ::"s"(lds),
                "v"(lvoff), "s"(r), "s"(soff), "s"(soff + xstep), "s"(soff + 2 * xstep), "s"(soff + 3 * xstep)
                : "memory");
        else
            asm volatile(
                "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
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

// Sum the per-wave partial results of a cooperative strip (coop) and store the 32 x D result as bf16 rows.
// acc[c][r] of lane (li, h): row li, feature 32c + acc_row(r, h).
// part (chunk of a long strip only): the work-group's sum goes there as fp32, register (c, r) of lane l at
// [(16c + r)*64 + l], instead of to the tensor.
template <int D>
__device__ __forceinline__ void store_rows_bf16(f32x16 (&acc)[D / 32], rsrc_t rO, int ld, int row0, bool coop, int w,
                                                int li, int h, float* lds, float* part = nullptr) {
    const int l = li + 32 * h;
    if (coop) {
        __syncthreads();  // lds is the memory of the wave-private tiles: every wavefront is done with them
        if (w > 0) {
#pragma unroll
            for (int c = 0; c < D / 32; ++c)
#pragma unroll
                for (int r = 0; r < 16; ++r) lds[(((w - 1) * (D / 32) + c) * 16 + r) * 64 + l] = acc[c][r];
        }
        __syncthreads();
        if (w > 0) return;
#pragma unroll
        for (int ww = 0; ww < BF16_WAVES - 1; ++ww)
#pragma unroll
            for (int c = 0; c < D / 32; ++c)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[c][r] += lds[((ww * (D / 32) + c) * 16 + r) * 64 + l];
        if (part) {
#pragma unroll
            for (int c = 0; c < D / 32; ++c)
#pragma unroll
                for (int r = 0; r < 16; ++r) part[(16 * c + r) * 64 + l] = acc[c][r];
            return;
        }
    }
    const int voff = (li * ld + 4 * h) * 2;
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            bf16x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = (__bf16)acc[c][4 * g + e];
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), rO, voff, row0 * ld * 2 + (32 * c + 8 * g) * 2, 0);
        }
}

// Work-group entry {a, b, c, d}.  a != b: strips a, b, c, d, one per wavefront (-1: none).  a == b: the four
// wavefronts walk chunk c of long strip a together (tiles c*chunk .. of the strip, `chunk` a launch parameter) and
// leave their sum in workspace slot d.
struct StripAssign {
    int strip, rank, step, chunk_id, slot;
    bool coop;
};
__device__ __forceinline__ StripAssign strip_of_wave(const int* __restrict__ wg_list, int g, int w) {
    const int4 e = reinterpret_cast<const int4*>(wg_list)[g];
    StripAssign s;
    s.coop = e.x == e.y;
    s.strip = s.coop ? e.x : (w == 0 ? e.x : w == 1 ? e.y : w == 2 ? e.z : e.w);
    s.rank = s.coop ? w : 0;
    s.step = s.coop ? BF16_WAVES : 1;
    s.chunk_id = s.coop ? e.z : 0;
    s.slot = s.coop ? e.w : -1;
    return s;
}
// floats per workspace slot: two 32 x D results (the column pass has dK and dV) and 64 row statistics
template <int D>
constexpr int bf16_slot_floats() { return 2 * 32 * D + 64; }

// -------------------------------------------------------------------------------------------------
// Forward: one sweep per block row with a lazily raised running maximum.
// -------------------------------------------------------------------------------------------------
// The LDS space of a forward work-group: the tile buffers of each wavefront (DmaTile; reused for the partial results
// of a shared strip) and the row statistics the wavefronts of a shared strip exchange.
template <int D>
struct Bf16FwdLds {
    typedef DmaTile<D> DT;
    __attribute__((aligned(16))) char t[BF16_WAVES][DT::WAVE];
    float m[BF16_WAVES][32], z[BF16_WAVES][32];
};

// One strip (or one chunk of a long strip, shared by the four wavefronts) per wavefront.
template <int D, bool MASK, bool ST>
__device__ __forceinline__ void bf16_fwd_strip(
    Bf16FwdLds<D>& lds, const StripAssign sa, int bh, int w, const __bf16* __restrict__ Q,
    const __bf16* __restrict__ K, const __bf16* __restrict__ V, const float* __restrict__ pen, __bf16* __restrict__ O,
    float* __restrict__ Lse, const int* __restrict__ trp, const int* __restrict__ tcol, int L, float scale,
    float* __restrict__ Part, int n_slots, int chunk, const Layouts& ly) {
    typedef DmaTile<D> DT;
    auto& lds_m = lds.m;
    auto& lds_z = lds.z;
    float* lds_o = reinterpret_cast<float*>(&lds.t[0][0]);  // partial results of a shared strip, after the tiles
    static_assert((BF16_WAVES - 1) * (D / 32) * 16 * 64 * 4 <= BF16_WAVES * DT::WAVE, "partial results fit");
    const int l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int I = sa.strip;
    const int cnt_all = trp[I + 1] - trp[I], tb = sa.chunk_id * chunk;
    const int t0 = trp[I] + tb, cnt = sa.coop ? min(chunk, cnt_all - tb) : cnt_all;
    const int nu = cnt > sa.rank ? (cnt - sa.rank + sa.step - 1) / sa.step : 0;
    float* part = sa.slot >= 0 ? Part + ((size_t)bh * n_slots + sa.slot) * bf16_slot_floats<D>() : nullptr;
    size_t ib, ob, ibytes, obytes;
    int ild, old_;
    bf16_head<ST, D>(ly.in, ly.H, bh, L, ib, ild, ibytes);
    bf16_head<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    const rsrc_t rQ = make_rsrc(Q + ib, ibytes);
    const rsrc_t rO = make_rsrc(O + ob, obytes);
    const u32x4 wK = rsrc_words(K + ib, ibytes), wV = rsrc_words(V + ib, ibytes);
    const u32x4 wM = rsrc_words(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
    const int r_voff = li * ild * 2 + h * D;
    const int t_bytes = 32 * ild * 2;
    const int d_voff = DT::voff(l, ild), d_xstep = DT::extra_step(ild);
    const char* Tw = lds.t[w];
    const unsigned lds_w = lds_address(Tw);
    const typename DT::RowAddr ra = DT::row_addr(li, h);
    const typename DT::TrAddr ta = DT::tr_addr(l);
    const float c2 = scale * LOG2E, pen_mul = -1.0f / scale;

    bf16x8 q[D / 16];
    ldb_rows<D>(rQ, r_voff, I * t_bytes, q);

    // Floor of the running maximum (the reference's max(-100, .) / max(0, .), models/block_attn.cu:52): any
    // value gives the same probabilities; 2^-100 keeps (L - n) * 2^-m finite in fp32 for empty rows.
    float m = MASK ? 0.f : -100.f, z = 0.f;
    f32x16 o[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) o[c] = splat16(0.f);

    constexpr int OPS = 2 * DT::NI + (MASK ? 1 : 0);
    auto tile_id = [&](int i) { return tcol[t0 + sa.rank + min(i, nu - 1) * sa.step]; };
    auto issue = [&](int J, int par) {  // key tile J -> buffer par
        const unsigned a = lds_w + par * DT::BUF;
        DT::load(wK, a, d_voff, J * t_bytes, d_xstep);
        DT::load(wV, a + DT::TILE, d_voff, J * t_bytes, d_xstep);
        if constexpr (MASK) dma_b32(wM, a + 2 * DT::TILE, l * 4, J * 128);
    };
    int Jq = 0;  // tile the next issue fetches, requested one tile ahead of that issue
    auto compute = [&](int par, int inext) {
        const char* Tk = Tw + par * DT::BUF;
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
        wait_lgkm0();  // the tile's operands are in registers: its buffer can take the tile after next
        if (inext >= 0) issue(Jq, par);
        Jq = tile_id(inext + 1);
        __builtin_amdgcn_sched_barrier(0);
        const f32x16 s = mma_feat_bf16<D>(kr, q, init);  // S^T: register = key, lane = query
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
        bf16x8 pb[2];
        pack16(p, pb);
        mma_tile_bf16<D>(vt, pb, o);  // O^T: register = feature, lane = query
        __builtin_amdgcn_sched_barrier(0);
    };
    settle(q);
    if (nu > 0) issue(tile_id(0), 0);
    if (nu > 1) issue(tile_id(1), 1);
    if (nu > 2) Jq = tile_id(2);
    for (int i = 0; i < nu; i += 2) {
        if (i + 1 < nu) wait_vm<OPS>();
        else wait_vm<0>();
        compute(0, i + 2 < nu ? i + 2 : -1);
        if (i + 1 >= nu) break;
        if (i + 2 < nu) wait_vm<OPS>();
        else wait_vm<0>();
        compute(1, i + 3 < nu ? i + 3 : -1);
    }
    z = half_swap_sum(z);
    if (sa.coop) {
        if (h == 0) {
            lds_m[w][li] = m;
            lds_z[w][li] = z;
        }
        __syncthreads();
        float M = lds_m[0][li];
#pragma unroll
        for (int ww = 1; ww < BF16_WAVES; ++ww) M = fmaxf(M, lds_m[ww][li]);
        float Z = 0.f;
#pragma unroll
        for (int ww = 0; ww < BF16_WAVES; ++ww) Z += lds_z[ww][li] * __builtin_amdgcn_exp2f(lds_m[ww][li] - M);
        const float f = __builtin_amdgcn_exp2f(m - M);
#pragma unroll
        for (int cc = 0; cc < D / 32; ++cc) o[cc] *= f;
        m = M;
        z = Z;
    }
    if (part) {  // chunk of a long strip: unnormalised sums relative to m; the merge kernel finishes the rows
        if (w == 0 && h == 0) {
            part[2 * 32 * D + li] = m;
            part[2 * 32 * D + 32 + li] = z;
        }
        store_rows_bf16<D>(o, rO, old_, I * 32, true, w, li, h, lds_o, part);
        return;
    }
    const int off_pattern = L - cnt_all * 32;
    if (off_pattern > 0) z += (float)off_pattern * __builtin_amdgcn_exp2f(-m);  // models/block_attn.cu:74
    const float rinv = 1.0f / z;
#pragma unroll
    for (int cc = 0; cc < D / 32; ++cc) o[cc] *= rinv;
    if (sa.rank == 0 && h == 0) Lse[(size_t)bh * L + I * 32 + li] = m + __builtin_amdgcn_logf(z);
    store_rows_bf16<D>(o, rO, old_, I * 32, sa.coop, w, li, h, lds_o);
}

template <int D, bool MASK, bool ST>
SPION_BF16_KERNEL(D == 32 ? (MASK ? 3 : 4) : 2) void bf16_fwd_kernel(
    const __bf16* __restrict__ Q, const __bf16* __restrict__ K, const __bf16* __restrict__ V,
    const float* __restrict__ pen, __bf16* __restrict__ O, float* __restrict__ Lse, const int* __restrict__ trp,
    const int* __restrict__ tcol, const int* __restrict__ wg_list, int n_wg, int L, int NB, float scale,
    float* __restrict__ Part, int n_slots, int chunk, Layouts ly) {
    __shared__ Bf16FwdLds<D> lds;
    const int item = xcd_remap(blockIdx.x, n_wg * NB);
    const int bh = item / n_wg;
    const int w = wave_index();
    const StripAssign sa = strip_of_wave(wg_list, item % n_wg, w);
    if (sa.strip < 0) return;  // only in entries of independent strips: no barrier is skipped
    bf16_fwd_strip<D, MASK, ST>(lds, sa, bh, w, Q, K, V, pen, O, Lse, trp, tcol, L, scale, Part, n_slots, chunk, ly);
}

// -------------------------------------------------------------------------------------------------
// Forward, two strips per wavefront: for masks of 64 x 64 blocks and larger, strips 2p and 2p+1 hold the same block
// columns, so one wavefront takes both: every K and V tile is fetched, copied to LDS and read back as an operand
// once for the two strips' chains, and the two softmax updates are independent instruction streams.  pair_list:
// four pair indices per work-group (-1: none); pairs whose strips are long enough to be cut into chunks stay with
// bf16_fwd_kernel.
// -------------------------------------------------------------------------------------------------
template <int D, bool MASK>
__device__ __forceinline__ void bf16_fwd_pair(
    Bf16FwdLds<D>& lds, int pr, int bh, int w, const __bf16* __restrict__ Q, const __bf16* __restrict__ K,
    const __bf16* __restrict__ V, const float* __restrict__ pen, __bf16* __restrict__ O, float* __restrict__ Lse,
    const int* __restrict__ trp, const int* __restrict__ tcol, int L, float scale) {
    typedef DmaTile<D> DT;
    const int l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int I = 2 * pr;
    const int t0 = trp[I], cnt = trp[I + 1] - t0;
    const size_t hb = (size_t)bh * L * D, hbytes = (size_t)L * D * 2;
    const rsrc_t rQ = make_rsrc(Q + hb, hbytes);
    const rsrc_t rO = make_rsrc(O + hb, hbytes);
    const u32x4 wK = rsrc_words(K + hb, hbytes), wV = rsrc_words(V + hb, hbytes);
    const u32x4 wM = rsrc_words(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
    const int r_voff = li * D * 2 + h * D;
    const int t_bytes = 32 * D * 2;
    const int d_voff = DT::voff(l, D);
    const char* Tw = lds.t[w];
    const unsigned lds_w = lds_address(Tw);
    const typename DT::RowAddr ra = DT::row_addr(li, h);
    const typename DT::TrAddr ta = DT::tr_addr(l);
    const float c2 = scale * LOG2E, pen_mul = -1.0f / scale;

    bf16x8 q0[D / 16], q1[D / 16];
    ldb_rows<D>(rQ, r_voff, I * t_bytes, q0);
    ldb_rows<D>(rQ, r_voff, (I + 1) * t_bytes, q1);
    float m0 = MASK ? 0.f : -100.f, z0 = 0.f, m1 = m0, z1 = 0.f;
    f32x16 o0[D / 32], o1[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        o0[c] = splat16(0.f);
        o1[c] = splat16(0.f);
    }
    auto update = [&](const f32x16& s, float& m, float& z, f32x16 (&o)[D / 32], bf16x8 (&pb)[2]) {
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
    constexpr int OPS = 2 * DT::NI + (MASK ? 1 : 0);
    auto tile_id = [&](int i) { return tcol[t0 + min(i, cnt - 1)]; };
    int Jq = 0;  // tile the next issue fetches, requested one tile ahead of that issue
    auto issue = [&](int J, int par) {
        const unsigned a = lds_w + par * DT::BUF;
        DT::load(wK, a, d_voff, J * t_bytes, 0);
        DT::load(wV, a + DT::TILE, d_voff, J * t_bytes, 0);
        if constexpr (MASK) dma_b32(wM, a + 2 * DT::TILE, l * 4, J * 128);
    };
    auto compute = [&](int par, int inext) {
        const char* Tk = Tw + par * DT::BUF;
        const char* Tv = Tk + DT::TILE;
        bf16x8 kr[D / 16], vt[D / 32][2];
        DT::get_rows(Tk, ra, kr);
        DT::get_tile_t(Tv, ta, vt);
        f32x16 init = splat16(0.f);
        if constexpr (MASK) {
            float pj[16];
            lds_get_rows(reinterpret_cast<const float*>(Tk + 2 * DT::TILE), 0, h, pj);
#pragma unroll
            for (int r = 0; r < 16; ++r) init[r] = pj[r] * pen_mul;
        }
        wait_lgkm0();
        if (inext >= 0) issue(Jq, par);
        Jq = tile_id(inext + 1);
        __builtin_amdgcn_sched_barrier(0);
        const f32x16 s0 = mma_feat_bf16<D>(kr, q0, init);
        const f32x16 s1 = mma_feat_bf16<D>(kr, q1, init);
        bf16x8 pb0[2], pb1[2];
        update(s0, m0, z0, o0, pb0);
        update(s1, m1, z1, o1, pb1);
        mma_tile_bf16<D>(vt, pb0, o0);
        mma_tile_bf16<D>(vt, pb1, o1);
        __builtin_amdgcn_sched_barrier(0);
    };
    settle(q0);
    settle(q1);
    if (cnt > 0) issue(tile_id(0), 0);
    if (cnt > 1) issue(tile_id(1), 1);
    if (cnt > 2) Jq = tile_id(2);
    for (int i = 0; i < cnt; i += 2) {
        if (i + 1 < cnt) wait_vm<OPS>();
        else wait_vm<0>();
        compute(0, i + 2 < cnt ? i + 2 : -1);
        if (i + 1 >= cnt) break;
        if (i + 2 < cnt) wait_vm<OPS>();
        else wait_vm<0>();
        compute(1, i + 3 < cnt ? i + 3 : -1);
    }
    const int off_pattern = L - cnt * 32;
    float* lds_unused = nullptr;
    auto finish = [&](float m, float z, f32x16 (&o)[D / 32], int strip) {
        z = half_swap_sum(z);
        if (off_pattern > 0) z += (float)off_pattern * __builtin_amdgcn_exp2f(-m);
        const float rinv = 1.0f / z;
#pragma unroll
        for (int cc = 0; cc < D / 32; ++cc) o[cc] *= rinv;
        if (h == 0) Lse[(size_t)bh * L + strip * 32 + li] = m + __builtin_amdgcn_logf(z);
        store_rows_bf16<D>(o, rO, D, strip * 32, false, w, li, h, lds_unused);
    };
    finish(m0, z0, o0, I);
    finish(m1, z1, o1, I + 1);
}

// Work-group list of the paired forward: entries {a, a, c, slot} are chunk c of long strip a, shared by the four
// wavefronts (bf16_fwd_strip; these entries come first), entries {p0, p1, p2, p3} four pairs of strips, one per
// wavefront (-1: none).  One launch for both kinds: the few work-groups of the long strips would otherwise set the
// length of a launch of their own (32 us for configuration 5).
template <int D, bool MASK>
SPION_BF16_KERNEL(2) void bf16_fwd_pair_kernel(
    const __bf16* __restrict__ Q, const __bf16* __restrict__ K, const __bf16* __restrict__ V,
    const float* __restrict__ pen, __bf16* __restrict__ O, float* __restrict__ Lse, const int* __restrict__ trp,
    const int* __restrict__ tcol, const int* __restrict__ list, int n_wg, int L, int NB, float scale,
    float* __restrict__ Part, int n_slots, int chunk) {
    __shared__ Bf16FwdLds<D> lds;
    const int item = xcd_remap(blockIdx.x, n_wg * NB);
    const int bh = item / n_wg;
    const int w = wave_index();
    const int4 e = reinterpret_cast<const int4*>(list)[item % n_wg];
    if (e.x == e.y) {  // uniform over the work-group
        const StripAssign sa = strip_of_wave(list, item % n_wg, w);
        bf16_fwd_strip<D, MASK, false>(lds, sa, bh, w, Q, K, V, pen, O, Lse, trp, tcol, L, scale, Part, n_slots, chunk,
                                       Layouts{});
        return;
    }
    const int pr = w == 0 ? e.x : w == 1 ? e.y : w == 2 ? e.z : e.w;
    if (pr < 0) return;
    bf16_fwd_pair<D, MASK>(lds, pr, bh, w, Q, K, V, pen, O, Lse, trp, tcol, L, scale);
}

// -------------------------------------------------------------------------------------------------
// Backward, row pass: g_i = dO_i . O_i, P and dP recomputed per tile, dS' = P*(dP - g), dQ += dS'.K_J;
// the 1/sqrt(d) is applied to the 32 x d result.  Stats receives {lse2, -g} of every strip (64 floats per strip:
// the 32 lse2 values, then the 32 -g values) for the column pass.
// K and V tiles go from global memory straight into one of two LDS buffers of the wavefront (DmaTile), two tiles
// ahead of the one being worked on.
// -------------------------------------------------------------------------------------------------
template <int D, bool MASK, bool ST>
SPION_BF16_KERNEL(D == 32 ? 3 : 2) void bf16_bwd_row_kernel(
    const __bf16* __restrict__ Q, const __bf16* __restrict__ K, const __bf16* __restrict__ V,
    const __bf16* __restrict__ dO, const __bf16* __restrict__ O, const float* __restrict__ Lse,
    const float* __restrict__ pen, float* __restrict__ Stats, __bf16* __restrict__ dQ, const int* __restrict__ trp,
    const int* __restrict__ tcol, const int* __restrict__ wg_list, int n_wg, int L, int NB, float scale,
    float* __restrict__ Part, int n_slots, int chunk, Layouts ly) {
    typedef DmaTile<D> DT;
    __shared__ __attribute__((aligned(16))) char lds_t[BF16_WAVES][DT::WAVE];
    float* lds_o = reinterpret_cast<float*>(&lds_t[0][0]);  // partial results of a shared strip, after the tiles
    static_assert((BF16_WAVES - 1) * (D / 32) * 16 * 64 * 4 <= BF16_WAVES * DT::WAVE, "partial results fit");
    const int item = xcd_remap(blockIdx.x, n_wg * NB);
    const int bh = item / n_wg;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const StripAssign sa = strip_of_wave(wg_list, item % n_wg, w);
    if (sa.strip < 0) return;
    const int I = sa.strip;
    const int cnt_all = trp[I + 1] - trp[I], tb = sa.chunk_id * chunk;
    const int t0 = trp[I] + tb, cnt = sa.coop ? min(chunk, cnt_all - tb) : cnt_all;
    const int nu = cnt > sa.rank ? (cnt - sa.rank + sa.step - 1) / sa.step : 0;
    float* part = sa.slot >= 0 ? Part + ((size_t)bh * n_slots + sa.slot) * bf16_slot_floats<D>() : nullptr;
    size_t ib, ob, gb, ibytes, obytes, gbytes;
    int ild, old_, gld;
    bf16_head<ST, D>(ly.in, ly.H, bh, L, ib, ild, ibytes);
    bf16_head<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    bf16_head<ST, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rQ = make_rsrc(Q + ib, ibytes);
    const rsrc_t rdO = make_rsrc(dO + ob, obytes), rO = make_rsrc(O + ob, obytes), rdQ = make_rsrc(dQ + gb, gbytes);
    const u32x4 wK = rsrc_words(K + ib, ibytes), wV = rsrc_words(V + ib, ibytes);
    const u32x4 wM = rsrc_words(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
    const int r_voff = li * ild * 2 + h * D, ro_voff = li * old_ * 2 + h * D;
    const int t_bytes = 32 * ild * 2;
    const int d_voff = DT::voff(l, ild), d_xstep = DT::extra_step(ild);
    const char* Tw = lds_t[w];
    const unsigned lds_w = lds_address(Tw);
    const typename DT::RowAddr ra = DT::row_addr(li, h);
    const typename DT::TrAddr ta = DT::tr_addr(l);
    const float c2 = scale * LOG2E, pen_mul = -1.0f / scale;

    bf16x8 q[D / 16], go[D / 16];
    ldb_rows<D>(rQ, r_voff, I * t_bytes, q);
    ldb_rows<D>(rdO, ro_voff, I * 32 * old_ * 2, go);
    float g = 0.f;
    {
        bf16x8 oo[D / 16];
        ldb_rows<D>(rO, ro_voff, I * 32 * old_ * 2, oo);
#pragma unroll
        for (int t = 0; t < D / 16; ++t)
#pragma unroll
            for (int e = 0; e < 8; ++e) g = fmaf((float)go[t][e], (float)oo[t][e], g);
        g = half_swap_sum(g);
    }
    const float lse = Lse[(size_t)bh * L + I * 32 + li];
    if (sa.rank == 0 && tb == 0) Stats[((size_t)bh * (L / 32) + I) * 64 + l] = h ? -g : lse;
    const f32x16 gneg = splat16(-g);

    f32x16 acc[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) acc[c] = splat16(0.f);
    // tile i of this wavefront -> buffer par
    constexpr int OPS = 2 * DT::NI + (MASK ? 1 : 0);
    auto tile_id = [&](int i) { return tcol[t0 + sa.rank + min(i, nu - 1) * sa.step]; };
    auto issue = [&](int J, int par) {
        const unsigned a = lds_w + par * DT::BUF;
        DT::load(wK, a, d_voff, J * t_bytes, d_xstep);
        DT::load(wV, a + DT::TILE, d_voff, J * t_bytes, d_xstep);
        if constexpr (MASK) dma_b32(wM, a + 2 * DT::TILE, l * 4, J * 128);
    };
    int Jq = 0;  // tile the next issue fetches, requested one tile ahead of that issue
    auto compute = [&](int par, int inext) {
        const char* Tk = Tw + par * DT::BUF;
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
        wait_lgkm0();  // the tile's operands are in registers: its buffer can take the tile after next
        if (inext >= 0) issue(Jq, par);
        Jq = tile_id(inext + 1);
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
    };
    settle(q);
    settle(go);
    settle(lse);
    if (nu > 0) issue(tile_id(0), 0);
    if (nu > 1) issue(tile_id(1), 1);
    if (nu > 2) Jq = tile_id(2);
    for (int i = 0; i < nu; i += 2) {
        if (i + 1 < nu) wait_vm<OPS>();
        else wait_vm<0>();
        compute(0, i + 2 < nu ? i + 2 : -1);
        if (i + 1 >= nu) break;
        if (i + 2 < nu) wait_vm<OPS>();
        else wait_vm<0>();
        compute(1, i + 3 < nu ? i + 3 : -1);
    }
#pragma unroll
    for (int c = 0; c < D / 32; ++c) acc[c] *= scale;
    store_rows_bf16<D>(acc, rdQ, gld, I * 32, sa.coop, w, li, h, lds_o, part);
}

// -------------------------------------------------------------------------------------------------
// Backward, column pass over the transposed tile index: dK_J = sum_I dS_IJ^T Q_I, dV_J = sum_I P_IJ^T dO_I.
// -------------------------------------------------------------------------------------------------
// Stats: {lse2, -g} of every strip as the row pass left them (64 floats per strip).  The Q and dO tiles and the
// tile's 64 statistics go from global memory straight into one of two LDS buffers of the wavefront (DmaTile).
template <int D, bool MASK, bool ST>
SPION_BF16_KERNEL(2) void bf16_bwd_col_kernel(
    const __bf16* __restrict__ Q, const __bf16* __restrict__ K, const __bf16* __restrict__ V,
    const __bf16* __restrict__ dO, const float* __restrict__ Stats,
    const float* __restrict__ pen, __bf16* __restrict__ dK, __bf16* __restrict__ dV, const int* __restrict__ tcp,
    const int* __restrict__ tcdesc, const int* __restrict__ wg_list, int n_wg, int L, int NB, float scale,
    float* __restrict__ Part, int n_slots, int chunk, Layouts ly) {
    typedef DmaTile<D> DT;
    __shared__ __attribute__((aligned(16))) char lds_t[BF16_WAVES][DT::WAVE];
    float* lds_o = reinterpret_cast<float*>(&lds_t[0][0]);  // partial results of a shared strip, after the tiles
    static_assert((BF16_WAVES - 1) * (D / 32) * 16 * 64 * 4 <= BF16_WAVES * DT::WAVE, "partial results fit");
    const int item = xcd_remap(blockIdx.x, n_wg * NB);
    const int bh = item / n_wg;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const StripAssign sa = strip_of_wave(wg_list, item % n_wg, w);
    if (sa.strip < 0) return;
    const int J = sa.strip;
    const int cnt_all = tcp[J + 1] - tcp[J], tb = sa.chunk_id * chunk;
    const int e0 = tcp[J] + tb, cnt = sa.coop ? min(chunk, cnt_all - tb) : cnt_all;
    const int nu = cnt > sa.rank ? (cnt - sa.rank + sa.step - 1) / sa.step : 0;
    float* part = sa.slot >= 0 ? Part + ((size_t)bh * n_slots + sa.slot) * bf16_slot_floats<D>() : nullptr;
    size_t ib, ob, gb, ibytes, obytes, gbytes;
    int ild, old_, gld;
    bf16_head<ST, D>(ly.in, ly.H, bh, L, ib, ild, ibytes);
    bf16_head<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    bf16_head<ST, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rK = make_rsrc(K + ib, ibytes), rV = make_rsrc(V + ib, ibytes);
    const rsrc_t rdK = make_rsrc(dK + gb, gbytes), rdV = make_rsrc(dV + gb, gbytes);
    const u32x4 wQ = rsrc_words(Q + ib, ibytes), wG = rsrc_words(dO + ob, obytes);
    const u32x4 wS = rsrc_words(Stats + (size_t)bh * (L / 32) * 64, (size_t)(L / 32) * 256);
    const int r_voff = li * ild * 2 + h * D;
    const int q_voff = DT::voff(l, ild), q_xstep = DT::extra_step(ild);
    const int o_voff = DT::voff(l, old_), o_xstep = DT::extra_step(old_);
    const char* Tw = lds_t[w];
    const unsigned lds_w = lds_address(Tw);
    const typename DT::RowAddr ra = DT::row_addr(li, h);
    const typename DT::TrAddr ta = DT::tr_addr(l);
    const float c2 = scale * LOG2E;

    bf16x8 k[D / 16], v[D / 16];
    ldb_rows<D>(rK, r_voff, J * 32 * ild * 2, k);
    ldb_rows<D>(rV, r_voff, J * 32 * ild * 2, v);
    f32x16 sinit = splat16(0.f);
    if constexpr (MASK) sinit = splat16(-pen[(size_t)bh * L + J * 32 + li] / scale);

    f32x16 ak[D / 32], av[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        ak[c] = splat16(0.f);
        av[c] = splat16(0.f);
    }
    const int4* __restrict__ desc = reinterpret_cast<const int4*>(tcdesc) + e0;
    constexpr int OPS = 2 * DT::NI + 1;
    auto tile_id = [&](int i) { return desc[sa.rank + min(i, nu - 1) * sa.step].x; };
    int Iq = 0;  // query tile the next issue fetches, requested one tile ahead of that issue
    auto issue = [&](int I, int par) {  // query tile I -> buffer par
        const unsigned a = lds_w + par * DT::BUF;
        DT::load(wQ, a, q_voff, I * 32 * ild * 2, q_xstep);
        DT::load(wG, a + DT::TILE, o_voff, I * 32 * old_ * 2, o_xstep);
        dma_b32(wS, a + 2 * DT::TILE, l * 4, I * 256);
    };
    // d = 64 has no registers for the transposed tiles while the first chains' operands are live: they are read
    // once the chains are issued, and the buffer is handed to the tile after next after that.
    constexpr bool DEEP = D == 32;
    auto compute = [&](int par, int inext) {
        const char* Tq = Tw + par * DT::BUF;
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
            wait_lgkm0();
            if (inext >= 0) issue(Iq, par);
            Iq = tile_id(inext + 1);
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
            wait_lgkm0();
            if (inext >= 0) issue(Iq, par);
            Iq = tile_id(inext + 1);
        }
        mma_tile_bf16<D>(qt, dsb, ak);  // dK^T: register = feature, lane = key
        mma_tile_bf16<D>(gt, pb, av);   // dV^T
        __builtin_amdgcn_sched_barrier(0);
    };
    settle(k);
    settle(v);
    if constexpr (MASK) settle(sinit[0]);
    if (nu > 0) issue(tile_id(0), 0);
    if (nu > 1) issue(tile_id(1), 1);
    if (nu > 2) Iq = tile_id(2);
    for (int i = 0; i < nu; i += 2) {
        if (i + 1 < nu) wait_vm<OPS>();
        else wait_vm<0>();
        compute(0, i + 2 < nu ? i + 2 : -1);
        if (i + 1 >= nu) break;
        if (i + 2 < nu) wait_vm<OPS>();
        else wait_vm<0>();
        compute(1, i + 3 < nu ? i + 3 : -1);
    }
#pragma unroll
    for (int c = 0; c < D / 32; ++c) ak[c] *= scale;
    store_rows_bf16<D>(ak, rdK, gld, J * 32, sa.coop, w, li, h, lds_o, part);
    if (sa.coop) __syncthreads();
    store_rows_bf16<D>(av, rdV, gld, J * 32, sa.coop, w, li, h, lds_o, part ? part + 32 * D : nullptr);
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
