// MFMA tile kernels of the sparse path (forward, backward row pass, backward column pass).
//
// What shapes these kernels (measured on MI355X): an fp32 MFMA and ordinary vector-ALU instructions
// do not overlap on a SIMD -- every VALU instruction adds its ~4-5 cycles (v_exp_f32 ~13) to the 64 cycles
// of each v_mfma_f32_32x32x2_f32 -- while memory instructions issue for free.  So the kernels
//   * do all addressing in scalar registers: buffer loads/stores with a per-head resource, one lane
//     offset computed once per kernel and a scalar byte offset per tile;
//   * fold constants into the MFMA chain instead of touching every element afterwards: the row maximum
//     (forward) or the softmax row sum g (backward) enters as the chain's initial accumulator, the
//     1/sqrt(d)*log2(e) factor is folded into Q once per work-group, the 1/sqrt(d) of the gradients is
//     applied once to the 32 x d result instead of to every tile;
//   * keep the per-CU vector-memory pipeline (TA/TCP tag lookups, the next bottleneck after the ALUs)
//     lean: a P tile, whose MFMA layout gives every lane 16-byte pieces of its own row (64 distinct
//     pieces per instruction), is read and written with one full 128-byte row per half-wave instead and
//     transposed through a wave-private LDS tile; LDS instructions do not compete with the MFMAs either;
//   * software-pipeline each wavefront's tile list (operands of the next tile are requested before the
//     current MFMA chain starts).  d = 32: the tiles go from global memory straight into wave-private LDS
//     (DmaTileF32 below), so nothing but LDS holds a tile in flight.  d = 64 loads into registers
//     (tile_pipeline): there loads are never issued under a branch between a load and its use -- the
//     compiler's s_waitcnt insertion merges conditional paths conservatively and would otherwise wait for
//     the loads just issued; when there is no next tile the current one is simply requested again, and a
//     wavefront's tiles are processed in pairs inside the loop (two register sets, no copies) with an odd
//     last tile after it: a prefetch whose only consumer sits in a conditional block would be sunk into
//     that block by the compiler, next to its use.
#pragma once
#include "tile_ops.h"

namespace spion {

#define SPION_TILE_KERNEL(W) __global__ __launch_bounds__(64 * (W)) __attribute__((amdgpu_waves_per_eu(2, 2)))

typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// Raw buffer resource over [p, p + bytes): out-of-range loads return 0, stores are dropped.
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, size_t bytes) {
    const unsigned n = bytes > 0xfffffff0ull ? 0xfffffff0u : (unsigned)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)n, 0x00020000);
}
__device__ __forceinline__ float ld1(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ f32x4 ld4(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
// Non-temporal forms for the P stream (read or written once per pass, far larger than the caches): P then
// does not displace the K/V/Q/dO tiles in L2.  Measured on the north star: -4 % on the whole step.
__device__ __forceinline__ float ld1_nt(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 2));
}
__device__ __forceinline__ f32x4 ld4_nt(rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 2));
}
// 128-bit buffer stores.  The hardware reads a store's data registers over several cycles after issue: a VALU write
// to one of them in the next two issue slots can reach the store (seen on MI355X as single stale 4-byte words, now
// and then).  The compiler keeps that distance, but only for stores whose soffset is not a register (with a register
// there it relies on an extra issue cycle that covers one of the two slots).  So the scalar part of the address is
// added to the lane offset and the soffset field stays zero: every hazard of the instruction is then the compiler's
// to handle, which inline assembly would hide from it (the wait states between a VALU write of a scalar register
// and a memory instruction that reads it, for one).  NT: non-temporal.
template <bool NT = false, typename X>
__device__ __forceinline__ void store_b128(X x, rsrc_t r, int voff, int soff) {
    static_assert(sizeof(X) == 16, "128-bit store");
    typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, x), r, voff + soff, 0, NT ? 2 : 0);
}
__device__ __forceinline__ void st4(rsrc_t r, int voff, int soff, f32x4 v) { store_b128(v, r, voff, soff); }

// Operand over the head dimension from a row-major [.][D] head slice: D/2 consecutive floats per lane.
// voff = ((lane%32)*D + (lane/32)*(D/2))*4 bytes, soff = byte offset of the tile's first row.
template <int D>
__device__ __forceinline__ void ldr_rows(rsrc_t r, int voff, int soff, float (&x)[D / 2]) {
#pragma unroll
    for (int q = 0; q < D / 8; ++q) {
        f32x4 v = ld4(r, voff, soff + 16 * q);
        x[4 * q + 0] = v.x;
        x[4 * q + 1] = v.y;
        x[4 * q + 2] = v.z;
        x[4 * q + 3] = v.w;
    }
}
// Same operand from a feature-major [D][L] head slice.  voff = ((lane/32)*(D/2)*L + lane%32)*4,
// soff = byte offset of the tile's first column.
template <int D>
__device__ __forceinline__ void ldr_cols(rsrc_t r, int L, int voff, int soff, float (&x)[D / 2]) {
#pragma unroll
    for (int s = 0; s < D / 2; ++s) x[s] = ld1(r, voff, soff + s * L * 4);
}
// B operand of a product over a tile's 32 rows from a row-major [.][D] head slice: slot (s, h) = tile row
// acc_row(s, h).  voff = (4*(lane/32)*D + lane%32)*4, soff = byte offset of the tile's first row.
template <int D>
__device__ __forceinline__ void ldr_tile_b(rsrc_t r, int voff, int soff, float (&x)[D / 32][16], int ld = D) {
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
#pragma unroll
        for (int s = 0; s < 16; ++s) x[c][s] = ld1(r, voff, soff + ((8 * (s >> 2) + (s & 3)) * ld + c * 32) * 4);
}
// 16 floats per lane laid out as 4 groups of 4 consecutive floats 8 apart (accumulator rows of one lane).
__device__ __forceinline__ void ldr_4x4(rsrc_t r, int voff, int soff, float (&x)[16]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        f32x4 v = ld4(r, voff, soff + 32 * g);
        x[4 * g + 0] = v.x;
        x[4 * g + 1] = v.y;
        x[4 * g + 2] = v.z;
        x[4 * g + 3] = v.w;
    }
}
__device__ __forceinline__ void str_4x4(rsrc_t r, int voff, int soff, const float (&x)[16]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) st4(r, voff, soff + 32 * g, (f32x4){x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]});
}

__device__ __forceinline__ void st1(rsrc_t r, int voff, int soff, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, voff, soff, 0);
}

// A 32 x 32 tile in the two register layouts a wavefront can hold it in:
//   "row owner": lane (li, h) holds M[li][acc_row(r, h)], r = 0..15  (the accumulator of M^T; A operand)
//   "col owner": lane (li, h) holds M[acc_row(r, h)][li]             (the accumulator of M; one full row per
//                                                                     half-wave and register: coalesced in memory)
// Global memory is touched in the col-owner layout; the wave-private LDS tile T (row stride TS floats)
// converts between the two.  Same-wave LDS accesses complete in order, so no barrier is involved.
constexpr int TS = 36;
// col-owner tile of a row-major array whose rows are `ld` floats apart: 16 b32 accesses.
// voff = (4*(lane/32)*ld + lane%32)*4, soff = byte offset of the tile's first element.
__device__ __forceinline__ void ldr_tile_cols(rsrc_t r, int voff, int soff, int ld, float (&x)[16]) {
#pragma unroll
    for (int q = 0; q < 16; ++q) x[q] = ld1(r, voff, soff + (8 * (q >> 2) + (q & 3)) * ld * 4);
}
__device__ __forceinline__ void str_tile_cols(rsrc_t r, int voff, int soff, int ld, const float (&x)[16]) {
#pragma unroll
    for (int q = 0; q < 16; ++q)  // only P tiles are written this way: non-temporal
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[q]), r, voff, soff + (8 * (q >> 2) + (q & 3)) * ld * 4, 2);
}
__device__ __forceinline__ void lds_put_cols(float* T, int li, int h, const float (&x)[16], int col0 = 0) {
#pragma unroll
    for (int q = 0; q < 16; ++q) T[acc_row(q, h) * TS + col0 + li] = x[q];
}
__device__ __forceinline__ void lds_get_cols(const float* T, int li, int h, float (&x)[16]) {
#pragma unroll
    for (int q = 0; q < 16; ++q) x[q] = T[acc_row(q, h) * TS + li];
}
__device__ __forceinline__ void lds_put_rows(float* T, int li, int h, const float (&x)[16]) {
#pragma unroll
    for (int g = 0; g < 4; ++g)
        *reinterpret_cast<f32x4*>(T + li * TS + 8 * g + 4 * h) = (f32x4){x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]};
}
__device__ __forceinline__ void lds_get_rows(const float* T, int li, int h, float (&x)[16]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(T + li * TS + 8 * g + 4 * h);
        x[4 * g + 0] = v.x;
        x[4 * g + 1] = v.y;
        x[4 * g + 2] = v.z;
        x[4 * g + 3] = v.w;
    }
}
// operand over 32 features of row li: x[s] = T[li][16*h + s]
__device__ __forceinline__ void lds_get_feat32(const float* T, int li, int h, float (&x)[16]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(T + li * TS + 16 * h + 4 * g);
        x[4 * g + 0] = v.x;
        x[4 * g + 1] = v.y;
        x[4 * g + 2] = v.z;
        x[4 * g + 3] = v.w;
    }
}

// "Linear" access to a 32 x 32 fp32 tile whose rows are `ld` floats apart: four 16-byte instructions in which
// lane l, instruction i touch row 8i + l/8, columns 4(l%8) .. +3 -- eight full 128-byte rows per instruction.
// The texture path spends about as long on a 4-byte-per-lane instruction as on half a 16-byte-per-lane one
// (measured: ~16 vs ~32 cycles per wavefront instruction), so a tile fetched this way costs half the
// 16 single-float instructions of the operand layouts; the operand layouts are then read from a wave-private
// LDS copy of the tile.
__device__ __forceinline__ int lin_voff(int l, int ld) { return ((l >> 3) * ld + 4 * (l & 7)) * 4; }
__device__ __forceinline__ void ldr_tile_lin(rsrc_t r, int voff, int soff, int ld, f32x4 (&raw)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = ld4(r, voff, soff + 32 * i * ld);
}
// Non-temporal: the P stream of the forward (written once, far larger than the caches) is kept from displacing
// the K/V tiles in L2; measured -11 % on the forward kernel, -1.3 % on the whole step.
__device__ __forceinline__ void str_tile_lin(rsrc_t r, int voff, int soff, int ld, const f32x4 (&raw)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) store_b128<true>(raw[i], r, voff, soff + 32 * i * ld);
}
// The same tile access for data a work-group reads back after writing it (partial sums kept in memory): loads are
// served by the L2 (device-scope policy: the vector L1 is not consulted), stores use the default policy.
__device__ __forceinline__ void ldr_tile_lin_l2(rsrc_t r, int voff, int soff, int ld, f32x4 (&raw)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
        raw[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff + 32 * i * ld, 16));
}
__device__ __forceinline__ void str_tile_lin_cached(rsrc_t r, int voff, int soff, int ld, const f32x4 (&raw)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) st4(r, voff, soff + 32 * i * ld, raw[i]);
}
__device__ __forceinline__ void lds_put_lin(float* T, int l, const f32x4 (&raw)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<f32x4*>(T + (8 * i + (l >> 3)) * TS + 4 * (l & 7)) = raw[i];
}
__device__ __forceinline__ void lds_get_lin(const float* T, int l, f32x4 (&raw)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = *reinterpret_cast<const f32x4*>(T + (8 * i + (l >> 3)) * TS + 4 * (l & 7));
}

// -------------------------------------------------------------------------------------------------
// 32 x 32 fp32 tiles that go from global memory straight into LDS (buffer loads with the LDS modifier): no
// registers hold a tile in flight, no ds_write is spent on it, and the path delivers about twice the bytes per
// clock of loads into registers.  One instruction moves 64 x 16 bytes to 1 KB of consecutive LDS addresses starting
// at M0 (+ the instruction's immediate offset, which is added to the global address as well): eight 128-byte tile
// rows.  Which 16-byte piece of a row a lane fetches is free, so the LDS image is unpadded rows with the pieces of
// row r permuted: piece c lies at position c ^ (r % 8).  One column of a given row across a half-wave (the 32 floats
// of a row, in some order) is then free of bank conflicts; a lane's own row in 16-byte pieces, which the 64-bank LDS
// serves sixteen lanes at a time, meets rows r and r + 8 on the same banks (8 cycles instead of 4 per instruction).
// A permutation without that (c ^ ((r/2 % 2)*4 + r/4 % 4)) was measured in these kernels and changes nothing: the LDS
// pipe is not what they wait for, and it costs a second lane offset and more address registers.
// The loads are inline assembly: the compiler neither counts them in its s_waitcnt bookkeeping nor knows that they
// write LDS.  The kernels wait for them with wait_vm<N> (N = loads issued after the ones waited for; loads return
// in order, and the compiler's own counts can then only wait longer than needed) and finish their LDS reads with
// wait_lgkm0 before a tile's space is requested again; both carry a memory clobber, so no LDS access moves across.
// Every block of loads starts with five wait states (s_mov to M0, s_nop 3): a scalar register written by a vector
// instruction -- v_readfirstlane, or v_readlane when the compiler restores a spilled scalar -- needs that distance
// before a memory instruction reads it, and the compiler, which adds it elsewhere, does not look inside assembly.
// -------------------------------------------------------------------------------------------------
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
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
// n = 0, 4, 8 or 12 operations may stay outstanding
__device__ __forceinline__ void wait_vm_upto(int n) {
    if (n >= 12) wait_vm<12>();
    else if (n >= 8) wait_vm<8>();
    else if (n >= 4) wait_vm<4>();
    else wait_vm<0>();
}
__device__ __forceinline__ void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// An empty use of registers.  The compiler waits for the loads that fill them before this point -- else it puts that
// wait at their first use inside a tile loop, as vmcnt(0), where it would also wait, on every iteration, for the
// tile loads just issued (which it does not know of).
__device__ __forceinline__ void settle(float x) { asm volatile("" ::"v"(x)); }
template <int N>
__device__ __forceinline__ void settle(const float (&x)[N]) {
#pragma unroll
    for (int t = 0; t < N; ++t) asm volatile("" ::"v"(x[t]));
}
// 64 floats (lane l: 4 bytes at voff) to 256 bytes of LDS
__device__ __forceinline__ void dma_b32(u32x4 r, unsigned lds, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dword %1, %2, %3 offen lds" ::"s"(lds), "v"(voff), "s"(r),
                 "s"(soff)
                 : "memory");
}
struct DmaTileF32 {
    static constexpr int TILE = 4096;  // bytes
    // Lane offset (bytes) into an array whose rows are `ld` floats apart: lane l fills position l % 8 of row l / 8
    // (+ 8 rows per instruction) with the piece that belongs there.
    __device__ static __forceinline__ int voff(int l, int ld) { return ((l >> 3) * ld + 4 * ((l & 7) ^ (l >> 3))) * 4; }
    // what the scalar offset advances by from one instruction to the next, beyond the 1024 its immediate adds
    __device__ static __forceinline__ int extra_step(int ld) { return 32 * ld - 1024; }
    template <bool NT = false>
    __device__ static __forceinline__ void load(u32x4 r, unsigned lds, int lvoff, int soff, int xstep) {
        if constexpr (NT)
            asm volatile(
                "s_mov_b32 m0, %0\n\ts_nop 3\n\t"
                "buffer_load_dwordx4 %1, %2, %3 offen nt lds\n\t"
                "buffer_load_dwordx4 %1, %2, %4 offen offset:1024 nt lds\n\t"
                "buffer_load_dwordx4 %1, %2, %5 offen offset:2048 nt lds\n\t"
                "buffer_load_dwordx4 %1, %2, %6 offen offset:3072 nt lds" ::"s"(lds),
                "v"(lvoff), "s"(r), "s"(soff), "s"(soff + xstep), "s"(soff + 2 * xstep), "s"(soff + 3 * xstep)
                : "memory");
        else
            asm volatile(
                "s_mov_b32 m0, %0\n\ts_nop 3\n\t"
                "buffer_load_dwordx4 %1, %2, %3 offen lds\n\t"
                "buffer_load_dwordx4 %1, %2, %4 offen offset:1024 lds\n\t"
                "buffer_load_dwordx4 %1, %2, %5 offen offset:2048 lds\n\t"
                "buffer_load_dwordx4 %1, %2, %6 offen offset:3072 lds" ::"s"(lds),
                "v"(lvoff), "s"(r), "s"(soff), "s"(soff + xstep), "s"(soff + 2 * xstep), "s"(soff + 3 * xstep)
                : "memory");
    }
    // Lane (li, h)'s pieces of its own row li: piece p0 + pstep*g, g = 0..3 (four 16-byte reads).
    struct Own {
        const char* a[4];
    };
    __device__ static __forceinline__ Own own_addr(const char* T, int li, int p0, int pstep) {
        Own x;
#pragma unroll
        for (int g = 0; g < 4; ++g) x.a[g] = T + li * 128 + 16 * ((p0 + pstep * g) ^ (li & 7));
        return x;
    }
    // (`off`: byte distance of the tile from the one the addresses were made for)
    __device__ static __forceinline__ void get(const Own& o, float (&x)[16], int off = 0) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(o.a[g] + off);
            x[4 * g + 0] = v.x;
            x[4 * g + 1] = v.y;
            x[4 * g + 2] = v.z;
            x[4 * g + 3] = v.w;
        }
    }
    // All eight pieces of the lane's own row li (32 floats).
    struct Own8 {
        const char* a[8];
    };
    __device__ static __forceinline__ Own8 own8_addr(const char* T, int li) {
        Own8 x;
#pragma unroll
        for (int g = 0; g < 8; ++g) x.a[g] = T + li * 128 + 16 * (g ^ (li & 7));
        return x;
    }
    __device__ static __forceinline__ void get32(const Own8& o, float (&x)[32]) {
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(o.a[g]);
            x[4 * g + 0] = v.x;
            x[4 * g + 1] = v.y;
            x[4 * g + 2] = v.z;
            x[4 * g + 3] = v.w;
        }
    }
    // Column li of the rows acc_row(q, h) = 8(q/4) + 4h + q%4, q = 0..15 (the tile in col-owner layout): one
    // address per q%4, the q/4 step is an immediate (rows 8 apart share their permutation).
    struct Cols {
        const char* a[4];
    };
    __device__ static __forceinline__ Cols cols_addr(const char* T, int li, int h) {
        Cols x;
#pragma unroll
        for (int b = 0; b < 4; ++b) x.a[b] = T + (4 * h + b) * 128 + 16 * ((li >> 2) ^ (4 * h + b)) + 4 * (li & 3);
        return x;
    }
    __device__ static __forceinline__ void get(const Cols& c, float (&x)[16], int off = 0) {
#pragma unroll
        for (int q = 0; q < 16; ++q) x[q] = *reinterpret_cast<const float*>(c.a[q & 3] + 1024 * (q >> 2) + off);
    }
    // Column li of the rows 16h + s, s = 0..15 (operand over 32 features from a feature-major tile).
    struct FeatCols {
        const char* a[8];
    };
    __device__ static __forceinline__ FeatCols featcols_addr(const char* T, int li, int h) {
        FeatCols x;
#pragma unroll
        for (int j = 0; j < 8; ++j) x.a[j] = T + (16 * h + j) * 128 + 16 * ((li >> 2) ^ j) + 4 * (li & 3);
        return x;
    }
    // column li of all 32 rows (addresses made with h = 0)
    __device__ static __forceinline__ void get32(const FeatCols& c, float (&x)[32]) {
#pragma unroll
        for (int s = 0; s < 32; ++s) x[s] = *reinterpret_cast<const float*>(c.a[s & 7] + 1024 * (s >> 3));
    }
    __device__ static __forceinline__ void get(const FeatCols& c, float (&x)[16], int off = 0) {
#pragma unroll
        for (int s = 0; s < 16; ++s) x[s] = *reinterpret_cast<const float*>(c.a[s & 7] + 1024 * (s >> 3) + off);
    }
};

// acc = init + A.B over the head dimension (chain of D/2 MFMA).
template <int D>
__device__ __forceinline__ f32x16 mma_feat_init(const float (&a)[D / 2], const float (&b)[D / 2], f32x16 init) {
    f32x16 acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], init, 0, 0, 0);
#pragma unroll
    for (int s = 1; s < D / 2; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc, 0, 0, 0);
    return acc;
}
template <int D>
__device__ __forceinline__ void mma_b(const float (&w)[16], const float (&x)[D / 32][16], f32x16 (&out)[D / 32]) {
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
#pragma unroll
        for (int s = 0; s < 16; ++s) out[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(w[s], x[c][s], out[c], 0, 0, 0);
}
__device__ __forceinline__ f32x16 splat16(float v) {
    return (f32x16){v, v, v, v, v, v, v, v, v, v, v, v, v, v, v, v};
}
__device__ __forceinline__ float max16(const f32x16& s, float m) {
#pragma unroll
    for (int r = 0; r < 16; r += 2) m = fmaxf(fmaxf(s[r], s[r + 1]), m);
    return m;
}

// Merge per-lane (max, sum-of-exp2) pairs of a row: the two half-waves, then the waves of the work-group.
template <int WAVES>
__device__ __forceinline__ void merge_max_sum(float& m, float& z, int w, int h, int li, float (*lds_m)[32],
                                              float (*lds_z)[32]) {
    float m2 = __shfl_xor(m, 32, 64), z2 = __shfl_xor(z, 32, 64);
    float M = fmaxf(m, m2);
    z = z * __builtin_amdgcn_exp2f(m - M) + z2 * __builtin_amdgcn_exp2f(m2 - M);
    m = M;
    if (WAVES > 1) {
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
}

// Where the [L][D] slice of head bh = b*H + hh of a [B][H][L][D] tensor lies when the tensor is a view of other
// memory (the [B][L][H*D] output of a projection, say): element (b, hh, i, f) at b*bstride + hh*hstride + i*ld + f
// floats.  One layout each for the inputs (Q, K, V), the outputs of the forward (Out, and dO with it) and the
// gradients (dQ, dK, dV).
struct HeadLayout {
    long long bstride;
    int hstride;
    int ld;
};
struct Layouts {
    HeadLayout in, out, grad;
    int H;
};
// Host side: true when no two elements of a [B][H][L][d] view with this layout share an address (required of every
// tensor the kernels write).  Heads either follow one another as whole blocks or are interleaved inside the rows.
inline bool layout_is_injective(const HeadLayout& y, int B, int H, int L, int d) {
    const long long row_span = (long long)(L - 1) * y.ld + d;
    const bool blocks = H == 1 || y.hstride >= row_span;
    const bool interleaved = y.hstride >= d && y.ld >= (long long)(H - 1) * y.hstride + d;
    if (!blocks && !interleaved) return false;
    const long long batch_span = (long long)(H - 1) * y.hstride + row_span;
    return B == 1 || y.bstride >= batch_span;
}
// ST = false: the heads are contiguous [NB][L][D] slices and every figure below is a compile-time constant.
template <bool ST, int D>
__device__ __forceinline__ void head_slice(const HeadLayout& y, int H, int bh, int L, size_t& base, int& ld,
                                           size_t& bytes) {
    if constexpr (ST) {
        const int b = bh / H, hh = bh - b * H;
        base = (size_t)b * y.bstride + (size_t)hh * y.hstride;
        ld = y.ld;
        bytes = ((size_t)(L - 1) * y.ld + D) * 4;
    } else {
        base = (size_t)bh * L * D;
        ld = D;
        bytes = (size_t)L * D * 4;
    }
}

// Work item -> (head, position in the strip order).  The heads are taken hc at a time; within such a group the
// items walk the strip order (long strips first) with the group's heads innermost, so that all long strips of the
// group start before any short one and the launch ends on short strips.  (Time stamps per work group on the north
// star shape, backward row pass: a CU's eight wavefront slots are 88 % filled over the launch, 5 % of the launch is
// the tail after the average CU's last work group ends, the dies end within 5 % of each other.)
__device__ __forceinline__ void item_to_head_strip(int item, int nstrips, int hc, int& head, int& pos) {
    const int per = nstrips * hc, g = item / per, r = item - g * per;
    head = g * hc + r % hc;
    pos = r / hc;
}

// Software-pipelined walk over the tiles first, first+step, ... (n of them) of one wavefront.
//   fetch(X, i)   requests everything tile #i (0-based position in this wavefront's list) needs into X;
//   compute(X, i) consumes it.  Positions past the end are clamped by the callers' fetch (valid, redundant).
template <class Pre, class Fetch, class Compute>
__device__ __forceinline__ void tile_pipeline(int n, Pre& a, Pre& b, Fetch fetch, Compute compute) {
    if (n <= 0) return;
    fetch(a, 0);
    int i = 0;
    for (; i + 1 < n; i += 2) {
        fetch(b, i + 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(a, i);
        __builtin_amdgcn_sched_barrier(0);
        fetch(a, i + 2);
        __builtin_amdgcn_sched_barrier(0);
        compute(b, i + 1);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (i < n) compute(a, i);
}

// -------------------------------------------------------------------------------------------------
// Forward, one work-group per (head, block row).  Logits are kept in the log2 domain:
// s' = (q.k) * log2(e)/sqrt(d) (- penalty*log2(e)), P = exp2(s' - m') / Z.
//
// MAXT > 0: every wavefront keeps the logit tiles of its share of the block row in registers (at most
// MAXT tiles), so each tile costs one QK^T chain and one PV chain.  MAXT == 0: two sweeps, the second
// recomputing the logits (any row length).  Ocache (optional): second copy of O for the backward.
// -------------------------------------------------------------------------------------------------
// KROW: the K operand is row-major [NB][L][D] (what a caller has before it makes the transposed copy the
// reference's ABI asks for) instead of feature-major [NB][D][L].  For d = 64 every lane then reads 128 bytes of
// its own row (one cache line per lane), which is slower than the feature-major form: the row-major entry points
// for contiguous heads therefore still transpose once; only the strided entry points use it.
// MAXT <= 6 at d = 32 (at most six logit tiles per wavefront) fits three wavefronts per SIMD: the buffer of the
// final reduction then shares the space of the wave-private tiles (a barrier in between).
// LONG (with MAXT > 0): a strip too long for the registers of its wavefronts takes the two sweeps inside the same
// launch, so the few long strips of a pattern -- global rows -- do not force the sweeps on all of them.  Always on
// at d = 64; at d = 32 it is an instantiation of its own, which leaves the kernel of the other patterns as it is.
template <int D, int WAVES, bool MASK, int MAXT, bool KROW = false, bool ST = false, bool LONG = D == 64>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(D == 32 && MAXT > 0 && MAXT <= 6 && !LONG ? 3 : 2, D == 32 && MAXT > 0 && MAXT <= 6 && !LONG ? 3 : 2)))
void tile_fwd_kernel(
    const float* __restrict__ Q, const float* __restrict__ Kt, const float* __restrict__ V,
    const float* __restrict__ pen, float* __restrict__ P, float* __restrict__ O, float* __restrict__ Ocache,
    const int* __restrict__ rdesc, const int* __restrict__ tcol, int L, int nbr,
    int NB, int nnz, float scale, int s0, int ns, int hc, Layouts ly) {
    static_assert(!ST || KROW, "strided heads: row-major operands");
    constexpr int KH = D / 2;
    // reduction buffer inside the tile space
    constexpr bool SHARE = (D == 32 ? MAXT > 0 && MAXT <= 6 : MAXT > 0) && WAVES > 1;
    __shared__ float lds_own[!SHARE && WAVES > 1 ? WAVES * (D / 32) * 16 * 64 : 1];
    __shared__ float lds_m[WAVES][32], lds_z[WAVES][32];
    // per wavefront: one padded tile (layout changes of P) and, with the logits in registers, 8 KB filled straight
    // from global memory (d = 32: two tiles in turn; d = 64: the two halves of one tile), plus key penalties
    constexpr int TW = 32 * TS + (MAXT > 0 ? 2 * 1024 + (MASK ? 128 : 0) : 0);
    __shared__ __attribute__((aligned(16))) float lds_t[WAVES][TW];
    static_assert(!SHARE || WAVES * TW >= WAVES * (D / 32) * 16 * 64, "the reduction fits in the tile space");
    float* lds = SHARE ? &lds_t[0][0] : lds_own;
    // this launch covers strips s0 .. s0+ns-1 of the longest-first order of every head
    const int item = xcd_remap(blockIdx.x, ns * NB);
    int bh, pos;
    item_to_head_strip(item, ns, hc, bh, pos);
    const int4 sd = reinterpret_cast<const int4*>(rdesc)[s0 + pos];  // {strip, first tile, tiles, P offset}
    const int I = sd.x, t0 = sd.y, cnt = sd.z;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int rn = cnt * 32;
    const size_t hb = (size_t)bh * L * D;
    size_t ib, ob, hbytes, obytes;
    int ild, old_;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    const rsrc_t rQ = make_rsrc(Q + ib, hbytes), rK = make_rsrc(Kt + ib, hbytes), rV = make_rsrc(V + ib, hbytes);
    const rsrc_t rP = make_rsrc(P + (size_t)bh * nnz, (size_t)nnz * 4);
    const rsrc_t rM = make_rsrc(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
    const int p_base = sd.w * 4;
    const int pc_voff = (4 * h * rn + li) * 4;  // col-owner access to a P tile
    const int col_voff = (h * KH * L + li) * 4;
    const int b_voff = (4 * h * ild + li) * 4;
    const int m_voff = 16 * h;
    float* T = lds_t[w];
    // P tile t of this block row: transpose to the col-owner layout and store full rows
    auto store_p = [&](const float (&p)[16], int t) {
        float pc[16];
        lds_put_rows(T, li, h, p);
        lds_get_cols(T, li, h, pc);
        str_tile_cols(rP, pc_voff, p_base + t * 128, rn, pc);
    };
    const float c2 = scale * LOG2E;

    float q[KH];
    ldr_rows<D>(rQ, (li * ild + h * KH) * 4, I * 32 * ild * 4, q);
#pragma unroll
    for (int s = 0; s < KH; ++s) q[s] *= c2;
    // operand over the head dimension of key tile J (lane = key, features h*D/2 ..)
    auto load_kf = [&](int J, float (&x)[KH]) {
        if constexpr (KROW) ldr_rows<D>(rK, (li * ild + h * KH) * 4, J * 32 * ild * 4, x);
        else ldr_cols<D>(rK, L, col_voff, J * 128, x);
    };

    // initial accumulator of a logit chain: minus the key penalties of the tile, in the log2 domain
    auto chain_init = [&](int J) -> f32x16 {
        if (!MASK) return splat16(0.f);
        float pj[16];
        ldr_4x4(rM, m_voff, J * 128, pj);
        f32x16 v;
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = -LOG2E * pj[r];
        return v;
    };

    float m = MASK ? 0.f : -100.f * LOG2E, z = 0.f;
    f32x16 o[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) o[c] = splat16(0.f);

    auto two_sweeps = [&]() {
        // ---- sweep 1: online row maximum and denominator -------------------------------------------
        const int nu = cnt > w ? (cnt - w + WAVES - 1) / WAVES : 0;  // tiles of this wavefront
        struct PreK {
            float k[KH];
            float pj[16];  // key penalties of the tile (MASK only)
        };
        auto fetch_k = [&](PreK& x, int i) {
            const int J = tcol[t0 + w + min(i, nu - 1) * WAVES];
            load_kf(J, x.k);
            if constexpr (MASK) ldr_4x4(rM, m_voff, J * 128, x.pj);
        };
        auto init_of = [&](const PreK& x, float shift) -> f32x16 {
            f32x16 v;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if constexpr (MASK) v[r] = -LOG2E * x.pj[r] - shift;
                else v[r] = -shift;
            }
            return v;
        };
        {
            PreK ka, kb;
            tile_pipeline(nu, ka, kb, fetch_k, [&](PreK& c, int) {
                f32x16 s = mma_feat_init<D>(c.k, q, init_of(c, 0.f));
                const float tm = max16(s, m);
                float zz = 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) zz += __builtin_amdgcn_exp2f(s[r] - tm);
                z = z * __builtin_amdgcn_exp2f(m - tm) + zz;
                m = tm;
            });
        }
        merge_max_sum<WAVES>(m, z, w, h, li, lds_m, lds_z);
        z += (float)(L - rn) * __builtin_amdgcn_exp2f(-m);
        const float rinv = 1.0f / z;
        // ---- sweep 2: logits again (minus the row maximum, folded into the chain), P, O ------------
        {
            struct PreKV {
                PreK k;
                float vb[D / 32][16];
            };
            PreKV xa, xb;
            tile_pipeline(
                nu, xa, xb,
                [&](PreKV& x, int i) {
                    fetch_k(x.k, i);
                    ldr_tile_b<D>(rV, b_voff, tcol[t0 + w + min(i, nu - 1) * WAVES] * 32 * ild * 4, x.vb, ild);
                },
                [&](PreKV& c, int i) {
                    f32x16 s = mma_feat_init<D>(c.k.k, q, init_of(c.k, m));
                    float p[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) p[r] = __builtin_amdgcn_exp2f(s[r]) * rinv;
                    store_p(p, w + i * WAVES);
                    mma_b<D>(p, c.vb, o);
                });
        }
    };
    constexpr bool FALLBACK = LONG && MAXT > 0;
    if constexpr (MAXT > 0) {
      if (FALLBACK && cnt > MAXT * WAVES) {
        two_sweeps();
      } else {
        const int nu = cnt > w ? (cnt - w + WAVES - 1) / WAVES : 0;  // tiles of this wavefront
        f32x16 S[MAXT];
        int Js[MAXT];  // tile ids of this wavefront, fetched up front (scalar loads, one wait)
#pragma unroll
        for (int u = 0; u < MAXT; ++u) Js[u] = u < nu ? tcol[t0 + w + u * WAVES] : 0;
        constexpr bool LIN = D == 32;
        // d = 32: K^T and V tiles go straight into two wave-private LDS tiles, alternately (tile u + 1 is requested
        // before the chain of tile u starts); P tiles leave as four 16-byte instructions after a layout change
        // in the padded tile.  Loads into LDS and the P stores share one in-order counter (wait_vm).
        const char* Tb = reinterpret_cast<const char*>(T + 32 * TS);
        const unsigned lb = LIN ? lds_address(Tb) : 0;
        // a K tile is 32 features x 32 keys with rows L floats apart, or (KROW) 32 keys x 32 features, contiguous
        const int KSTEP = KROW ? 32 * ild * 4 : 128;
        const int kld = KROW ? ild : L;
        const int plin = lin_voff(l, rn);
        if constexpr (LIN) {
            const u32x4 wK = rsrc_words(Kt + ib, hbytes);
            const u32x4 wM = rsrc_words(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
            const int kl = DmaTileF32::voff(l, kld), kx = DmaTileF32::extra_step(kld);
            const auto a_k0 = [&] {
                if constexpr (KROW) return DmaTileF32::own_addr(Tb, li, 4 * h, 1);
                else return DmaTileF32::featcols_addr(Tb, li, h);
            }();
            // the key penalties of a tile travel with it (64 floats, of which the first 32 are the tile's)
            const char* Tm = Tb + 2 * DmaTileF32::TILE + 16 * h;
            constexpr int KOPS = MASK ? 5 : 4;
            auto issue_k = [&](int u) {
                DmaTileF32::load(wK, lb + (u & 1) * DmaTileF32::TILE, kl, Js[u] * KSTEP, kx);
                if constexpr (MASK) dma_b32(wM, lb + 2 * DmaTileF32::TILE + (u & 1) * 256, l * 4, Js[u] * 128);
            };
            if (nu > 0) issue_k(0);
#pragma unroll
            for (int u = 0; u < MAXT; ++u) {
                if (u < nu) {
                    if (u + 1 < MAXT && u + 1 < nu) {
                        issue_k(u + 1 < MAXT ? u + 1 : u);
                        wait_vm<KOPS>();
                    } else {
                        wait_vm<0>();
                    }
                    float kf[KH];
                    DmaTileF32::get(a_k0, kf, (u & 1) * DmaTileF32::TILE);
                    f32x16 init = splat16(0.f);
                    if constexpr (MASK) {  // minus the key penalties, in the log2 domain
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const f32x4 v = *reinterpret_cast<const f32x4*>(Tm + (u & 1) * 256 + 32 * g);
                            init[4 * g + 0] = -LOG2E * v.x;
                            init[4 * g + 1] = -LOG2E * v.y;
                            init[4 * g + 2] = -LOG2E * v.z;
                            init[4 * g + 3] = -LOG2E * v.w;
                        }
                    }
                    wait_lgkm0();  // the tile's space is requested again one iteration on
                    __builtin_amdgcn_sched_barrier(0);
                    S[u] = mma_feat_init<D>(kf, q, init);
                    m = max16(S[u], m);
                }
            }
        } else {
            // d = 64: a K tile is two 4 KB tiles (features 0..31 and 32..63) in one place; the operand of tile u is
            // read out into registers, then the place is requested for tile u + 1, which has the chain to arrive.
            static_assert(D == 64, "head dimension 32 or 64");
            const u32x4 wK = rsrc_words(Kt + ib, hbytes);
            const u32x4 wM = rsrc_words(MASK ? pen + (size_t)bh * L : pen, MASK ? (size_t)L * 4 : 0);
            const int kl = DmaTileF32::voff(l, kld), kx = DmaTileF32::extra_step(kld);
            const int KHALF = KROW ? 128 : 32 * L * 4;
            const unsigned lb64 = lds_address(Tb);
            const auto a_k = [&] {  // features 32h .. 32h+31 of key li: the half-wave's own tile
                if constexpr (KROW) return DmaTileF32::own8_addr(Tb + h * DmaTileF32::TILE, li);
                else return DmaTileF32::featcols_addr(Tb + h * DmaTileF32::TILE, li, 0);
            }();
            const char* Tm = Tb + 2 * DmaTileF32::TILE + 16 * h;
            auto issue_k = [&](int u) {
                DmaTileF32::load(wK, lb64, kl, Js[u] * KSTEP, kx);
                DmaTileF32::load(wK, lb64 + DmaTileF32::TILE, kl, Js[u] * KSTEP + KHALF, kx);
                if constexpr (MASK) dma_b32(wM, lb64 + 2 * DmaTileF32::TILE, l * 4, Js[u] * 128);
            };
            if (nu > 0) issue_k(0);
#pragma unroll
            for (int u = 0; u < MAXT; ++u) {
                if (u < nu) {
                    wait_vm<0>();
                    float kf[KH];
                    DmaTileF32::get32(a_k, kf);
                    f32x16 init = splat16(0.f);
                    if constexpr (MASK) {  // minus the key penalties, in the log2 domain
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const f32x4 v = *reinterpret_cast<const f32x4*>(Tm + 32 * g);
                            init[4 * g + 0] = -LOG2E * v.x;
                            init[4 * g + 1] = -LOG2E * v.y;
                            init[4 * g + 2] = -LOG2E * v.z;
                            init[4 * g + 3] = -LOG2E * v.w;
                        }
                    }
                    wait_lgkm0();
                    if (u + 1 < MAXT && u + 1 < nu) issue_k(u + 1 < MAXT ? u + 1 : u);
                    __builtin_amdgcn_sched_barrier(0);
                    S[u] = mma_feat_init<D>(kf, q, init);
                    m = max16(S[u], m);
                }
            }
        }
        // Exponentials relative to this wavefront's own maximum; one merge of (maximum, sum) pairs over the
        // half-waves and wavefronts then gives the row's maximum M and denominator, and the probabilities
        // are the exponentials times 2^(m - M) / Z.
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
        if (WAVES > 1) {
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
        z += (float)(L - rn) * __builtin_amdgcn_exp2f(-m);
        // +inf denominator -> 0 -> P = 0, as in the reference
        const float rinv = __builtin_amdgcn_exp2f(m_own - m) * (1.0f / z);

        if constexpr (LIN) {
            // V tiles the same way: request u + 2 goes out when tile u has been read.  What was issued after the
            // loads of tile u when its turn comes: the loads of tile u + 1 (if any), and the P stores of the one
            // or two tiles before it.
            const u32x4 wV = rsrc_words(V + ib, hbytes);
            const int vl = DmaTileF32::voff(l, ild), vx = DmaTileF32::extra_step(ild);
            const auto a_v0 = DmaTileF32::cols_addr(Tb, li, h);
            auto issue_v = [&](int u) {
                DmaTileF32::load(wV, lb + (u & 1) * DmaTileF32::TILE, vl, Js[u] * 32 * ild * 4, vx);
            };
            if (nu > 0) issue_v(0);
            if (MAXT > 1 && nu > 1) issue_v(1 < MAXT ? 1 : 0);
#pragma unroll
            for (int u = 0; u < MAXT; ++u) {
                if (u < nu) {
                    const int t = w + u * WAVES;
                    const int stores = u == 0 ? 0 : u == 1 ? 4 : 8;  // P stores issued after V tile u was requested
                    wait_vm_upto(stores + (u + 1 < MAXT && u + 1 < nu ? 4 : 0));
                    float p[16], vb[1][16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) p[r] = S[u][r] * rinv;
                    lds_put_rows(T, li, h, p);
                    DmaTileF32::get(a_v0, vb[0], (u & 1) * DmaTileF32::TILE);
                    f32x4 pl[4];
                    lds_get_lin(T, l, pl);
                    wait_lgkm0();
                    if (u + 2 < MAXT && u + 2 < nu) issue_v(u + 2 < MAXT ? u + 2 : u);
                    __builtin_amdgcn_sched_barrier(0);
                    mma_b<D>(p, vb, o);
                    str_tile_lin(rP, plin, p_base + t * 128, rn, pl);
                }
            }
        } else {
            // d = 64: the V tiles take the place of the K tiles, one tile ahead; after the loads of tile u only the
            // four P stores of tile u - 1 were issued.
            const u32x4 wV = rsrc_words(V + ib, hbytes);
            const int vl = DmaTileF32::voff(l, ild), vx = DmaTileF32::extra_step(ild);
            const unsigned lb64 = lds_address(Tb);
            const auto a_v = DmaTileF32::cols_addr(Tb, li, h);
            auto issue_v = [&](int u) {
                DmaTileF32::load(wV, lb64, vl, Js[u] * 32 * ild * 4, vx);
                DmaTileF32::load(wV, lb64 + DmaTileF32::TILE, vl, Js[u] * 32 * ild * 4 + 128, vx);
            };
            if (nu > 0) issue_v(0);
#pragma unroll
            for (int u = 0; u < MAXT; ++u) {
                if (u < nu) {
                    const int t = w + u * WAVES;
                    wait_vm_upto(u == 0 ? 0 : 4);
                    float p[16], vb[2][16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) p[r] = S[u][r] * rinv;
                    lds_put_rows(T, li, h, p);
                    DmaTileF32::get(a_v, vb[0]);
                    DmaTileF32::get(a_v, vb[1], DmaTileF32::TILE);
                    f32x4 pl[4];
                    lds_get_lin(T, l, pl);
                    wait_lgkm0();
                    if (u + 1 < MAXT && u + 1 < nu) issue_v(u + 1 < MAXT ? u + 1 : u);
                    __builtin_amdgcn_sched_barrier(0);
                    mma_b<D>(p, vb, o);
                    str_tile_lin(rP, plin, p_base + t * 128, rn, pl);
                }
            }
        }
      }
    } else {
        two_sweeps();
    }
    if constexpr (SHARE) __syncthreads();  // every wavefront is done with its tiles
    if (!ST && Ocache) reduce_store2<D, WAVES>(o, O + hb, Ocache + hb, I * 32, w, li, h, lds);
    else reduce_store<D, WAVES>(o, O + ob, I * 32, w, li, h, lds, old_);
}

// -------------------------------------------------------------------------------------------------
// Backward, row pass.  HAVE_O: the handle kept O of the matching forward, so g_i = dO_i . O_i is known up
// front; otherwise a first sweep accumulates g_i = sum_j dP_ij P_ij.  Main sweep per tile:
// dP^T - g = V_J.dO_I^T chain started from -g, dS' = (dP - g)*P, dQ += dS'.K_J; the 1/sqrt(d) is applied to
// the 32 x d result.  G receives -g for the column pass.
// -------------------------------------------------------------------------------------------------
// VROW: the V operand is row-major [NB][L][D] instead of feature-major [NB][D][L].
template <int D, int WAVES, bool HAVE_O, bool VROW = false, bool ST = false>
SPION_TILE_KERNEL(WAVES) void tile_bwd_row_kernel(
    const float* __restrict__ K, const float* __restrict__ Vt, const float* __restrict__ P,
    const float* __restrict__ dO, const float* __restrict__ Ocache, float* __restrict__ G,
    float* __restrict__ dQ, const int* __restrict__ rdesc, const int* __restrict__ tcol,
    int L, int nbr, int NB, int nnz, float scale, int hc, Layouts ly, int s0, int ns) {
    static_assert(!ST || (VROW && HAVE_O), "strided heads: row-major operands, Out given");
    constexpr int KH = D / 2;
    // LDS of a wavefront: the V, P and K tiles of one pattern tile, 4 KB per 32 features.  d = 64 needs 20 KB, which
    // eight wavefronts per CU fill to the last byte: the buffer of the final reduction and the partial row sums
    // of the first sweep then lie inside that space (CARVE), each separated from the tiles by a barrier.
    constexpr bool CARVE = D == 64;
    constexpr int WB = (1 + 2 * (D / 32)) * DmaTileF32::TILE;
    constexpr int RED = WAVES > 1 ? WAVES * (D / 32) * 16 * 64 * 4 : 0;
    static_assert(!CARVE || RED <= WAVES * WB, "the reduction fits in the tile space");
    __shared__ __attribute__((aligned(16))) char smem[CARVE ? WAVES * WB : WAVES * WB + RED + WAVES * 128];
    float* lds = reinterpret_cast<float*>(CARVE ? smem : smem + WAVES * WB);
    auto lds_g = [&](int ww) {
        return reinterpret_cast<float*>(CARVE ? smem + ww * WB + WB - 128 : smem + WAVES * WB + RED + ww * 128);
    };
    // Last head first: the forward wrote P front to back, so its tail is what the memory-side cache still holds.
    // This launch covers strips s0 .. s0+ns-1 of every head's strip order.
    const int item = xcd_remap(blockIdx.x, ns * NB);
    int bh, pos;
    item_to_head_strip(item, ns, hc, bh, pos);
    bh = NB - 1 - bh;
    const int4 sd = reinterpret_cast<const int4*>(rdesc)[s0 + pos];  // strips longest first: {strip, first tile, tiles, P offset}
    const int I = sd.x, t0 = sd.y, cnt = sd.z;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    const int rn = cnt * 32;
    const int nu = cnt > w ? (cnt - w + WAVES - 1) / WAVES : 0;  // tiles of this wavefront
    size_t ib, ob, gb, hbytes, obytes, gbytes;
    int ild, old_, gld;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    head_slice<ST, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rK = make_rsrc(K + ib, hbytes), rV = make_rsrc(Vt + ib, hbytes), rdO = make_rsrc(dO + ob, obytes);
    const rsrc_t rP = make_rsrc(P + (size_t)bh * nnz, (size_t)nnz * 4);
    const int p_base = sd.w * 4;
    const int pc_voff = (4 * h * rn + li) * 4;  // col-owner access to a P tile
    const int col_voff = (h * KH * L + li) * 4;
    const int b_voff = (4 * h * ild + li) * 4;
    const int r_voff = (li * ild + h * KH) * 4, ro_voff = (li * old_ + h * KH) * 4;
    float* T = reinterpret_cast<float*>(smem + w * WB);
    // P tile as loaded (col owner) -> row-owner layout, the one dP^T comes in
    auto p_rows = [&](const float (&pc)[16], float (&pr)[16]) {
        lds_put_cols(T, li, h, pc);
        lds_get_rows(T, li, h, pr);
    };

    float go[KH];
    ldr_rows<D>(rdO, ro_voff, I * 32 * old_ * 4, go);

    float g = 0.f;
    if (HAVE_O) {
        float oo[KH];
        ldr_rows<D>(make_rsrc(Ocache + ob, obytes), ro_voff, I * 32 * old_ * 4, oo);
#pragma unroll
        for (int s = 0; s < KH; ++s) g = fmaf(go[s], oo[s], g);
        g += __shfl_xor(g, 32, 64);
    } else {
        struct PreG {
            float vt[KH];
            float pv[16];
        };
        PreG xa, xb;
        tile_pipeline(
            nu, xa, xb,
            [&](PreG& x, int i) {
                const int t = w + min(i, nu - 1) * WAVES;
                if constexpr (VROW) ldr_rows<D>(rV, r_voff, tcol[t0 + t] * 32 * ild * 4, x.vt);
                else ldr_cols<D>(rV, L, col_voff, tcol[t0 + t] * 128, x.vt);
                ldr_tile_cols(rP, pc_voff, p_base + t * 128, rn, x.pv);
            },
            [&](PreG& c, int) {
                float pr[16];
                p_rows(c.pv, pr);
                f32x16 dp = mma_feat_init<D>(c.vt, go, splat16(0.f));
#pragma unroll
                for (int r = 0; r < 16; ++r) g = fmaf(dp[r], pr[r], g);
            });
        g += __shfl_xor(g, 32, 64);
        if (WAVES > 1) {
            if (h == 0) lds_g(w)[li] = g;
            __syncthreads();
            g = 0.f;
#pragma unroll
            for (int ww = 0; ww < WAVES; ++ww) g += lds_g(ww)[li];
            if constexpr (CARVE) __syncthreads();  // the partial sums lie where tiles are about to land
        }
    }
    if (w == 0 && h == 0) G[(size_t)bh * L + I * 32 + li] = -g;
    const f32x16 gneg = splat16(-g);

    f32x16 acc[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) acc[c] = splat16(0.f);
    if constexpr (D == 32) {
        // The V^T, P and K tiles of a tile go straight into wave-private LDS (twelve instructions, no registers in
        // flight); the operands of tile i are read out of LDS into registers, then the same space is requested for
        // tile i + 1, whose loads have the two chains of tile i to arrive.
        const char* Tv = reinterpret_cast<const char*>(T);
        const char* Tp = Tv + DmaTileF32::TILE;
        const char* Tk = Tv + 2 * DmaTileF32::TILE;
        const unsigned lv = lds_address(Tv), lp = lv + DmaTileF32::TILE, lk = lv + 2 * DmaTileF32::TILE;
        const u32x4 wV = rsrc_words(Vt + ib, hbytes), wK = rsrc_words(K + ib, hbytes);
        const u32x4 wP = rsrc_words(P + (size_t)bh * nnz, (size_t)nnz * 4);
        const int VSTEP = VROW ? 32 * ild * 4 : 128;
        const int vld = VROW ? ild : L;
        const int vl = DmaTileF32::voff(l, vld), pl = DmaTileF32::voff(l, rn), kl = DmaTileF32::voff(l, ild);
        const int vx = DmaTileF32::extra_step(vld), px = DmaTileF32::extra_step(rn), kx = DmaTileF32::extra_step(ild);
        const auto a_v = [&] {
            if constexpr (VROW) return DmaTileF32::own_addr(Tv, li, 4 * h, 1);
            else return DmaTileF32::featcols_addr(Tv, li, h);
        }();
        const auto a_p = DmaTileF32::own_addr(Tp, li, h, 2);
        const auto a_k = DmaTileF32::cols_addr(Tk, li, h);
        auto issue = [&](int t, int J) {
            DmaTileF32::load(wV, lv, vl, J * VSTEP, vx);
            DmaTileF32::load<true>(wP, lp, pl, p_base + t * 128, px);
            DmaTileF32::load(wK, lk, kl, J * 32 * ild * 4, kx);
        };
        if (nu > 0) {
            issue(w, tcol[t0 + w]);
            int Jn = tcol[t0 + w + (nu > 1 ? WAVES : 0)];
            for (int i = 0; i < nu; ++i) {
                const int Jnn = tcol[t0 + w + min(i + 2, nu - 1) * WAVES];  // index of the tile after the next
                wait_vm<0>();
                float vt[16], pr[16], kb[1][16];
                DmaTileF32::get(a_v, vt);
                DmaTileF32::get(a_p, pr);
                DmaTileF32::get(a_k, kb[0]);
                wait_lgkm0();
                if (i + 1 < nu) issue(w + (i + 1) * WAVES, Jn);
                Jn = Jnn;
                __builtin_amdgcn_sched_barrier(0);
                f32x16 dp = mma_feat_init<D>(vt, go, gneg);  // dp[r] = dO_i . v_j - g_i
                float ds[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) ds[r] = dp[r] * pr[r];
                mma_b<D>(ds, kb, acc);
            }
        }
    } else {
        // d = 64, the same schedule: the V and K tiles are two 4 KB tiles each (features 0..31 and 32..63), the P
        // tile one; twenty instructions a tile.
        static_assert(D == 64, "head dimension 32 or 64");
        const char* Tv = reinterpret_cast<const char*>(T);
        const char* Tk = Tv + 2 * DmaTileF32::TILE;
        const char* Tp = Tv + 4 * DmaTileF32::TILE;
        const unsigned lv = lds_address(Tv), lk = lv + 2 * DmaTileF32::TILE, lp = lv + 4 * DmaTileF32::TILE;
        const u32x4 wV = rsrc_words(Vt + ib, hbytes), wK = rsrc_words(K + ib, hbytes);
        const u32x4 wP = rsrc_words(P + (size_t)bh * nnz, (size_t)nnz * 4);
        // V: feature-major, the halves are 32 rows of L floats apart; row-major, 32 floats apart inside a row
        const int VSTEP = VROW ? 32 * ild * 4 : 128, VHALF = VROW ? 128 : 32 * L * 4;
        const int vld = VROW ? ild : L;
        const int vl = DmaTileF32::voff(l, vld), pl = DmaTileF32::voff(l, rn), kl = DmaTileF32::voff(l, ild);
        const int vx = DmaTileF32::extra_step(vld), px = DmaTileF32::extra_step(rn), kx = DmaTileF32::extra_step(ild);
        // operand of the first chain: features 32h .. 32h+31 of key li, i.e. the half-wave's own V tile
        const auto a_v = [&] {
            if constexpr (VROW) return DmaTileF32::own8_addr(Tv + h * DmaTileF32::TILE, li);
            else return DmaTileF32::featcols_addr(Tv + h * DmaTileF32::TILE, li, 0);
        }();
        const auto a_p = DmaTileF32::own_addr(Tp, li, h, 2);
        const auto a_k = DmaTileF32::cols_addr(Tk, li, h);
        auto issue = [&](int t, int J) {
            DmaTileF32::load(wV, lv, vl, J * VSTEP, vx);
            DmaTileF32::load(wV, lv + DmaTileF32::TILE, vl, J * VSTEP + VHALF, vx);
            DmaTileF32::load<true>(wP, lp, pl, p_base + t * 128, px);
            DmaTileF32::load(wK, lk, kl, J * 32 * ild * 4, kx);
            DmaTileF32::load(wK, lk + DmaTileF32::TILE, kl, J * 32 * ild * 4 + 128, kx);
        };
        if (nu > 0) {
            issue(w, tcol[t0 + w]);
            int Jn = tcol[t0 + w + (nu > 1 ? WAVES : 0)];
            for (int i = 0; i < nu; ++i) {
                const int Jnn = tcol[t0 + w + min(i + 2, nu - 1) * WAVES];  // index of the tile after the next
                wait_vm<0>();
                float vt[KH], pr[16], kb[2][16];
                DmaTileF32::get32(a_v, vt);
                DmaTileF32::get(a_p, pr);
                DmaTileF32::get(a_k, kb[0]);
                DmaTileF32::get(a_k, kb[1], DmaTileF32::TILE);
                wait_lgkm0();
                if (i + 1 < nu) issue(w + (i + 1) * WAVES, Jn);
                Jn = Jnn;
                __builtin_amdgcn_sched_barrier(0);
                f32x16 dp = mma_feat_init<D>(vt, go, gneg);  // dp[r] = dO_i . v_j - g_i
                float ds[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) ds[r] = dp[r] * pr[r];
                mma_b<D>(ds, kb, acc);
            }
        }
    }
    if constexpr (CARVE && WAVES > 1) __syncthreads();  // every wavefront is done with its tiles
#pragma unroll
    for (int c = 0; c < D / 32; ++c) acc[c] *= scale;
    reduce_store<D, WAVES>(acc, dQ + gb, I * 32, w, li, h, lds, gld);
}

// -------------------------------------------------------------------------------------------------
// Backward, column pass, one work-group per (head, block column): dK_J = sum_I dS_IJ^T Q_I,
// dV_J = sum_I P_IJ^T dO_I over the transposed tile index; dP - g is recomputed per tile by a chain
// started from the stored -g, the 1/sqrt(d) of dK is applied to the 32 x d result.
// -------------------------------------------------------------------------------------------------
// VROW: as in the row pass.
template <int D, int WAVES, bool VROW = false, bool ST = false>
SPION_TILE_KERNEL(WAVES) void tile_bwd_col_kernel(
    const float* __restrict__ Q, const float* __restrict__ Vt, const float* __restrict__ P,
    const float* __restrict__ dO, const float* __restrict__ G, float* __restrict__ dK, float* __restrict__ dV,
    const int* __restrict__ cdesc, const int* __restrict__ tcdesc, int L, int nbr, int NB, int nnz, float scale,
    int hc, Layouts ly, int s0, int ns) {
    static_assert(!ST || VROW, "strided heads: row-major operands");
    constexpr int KH = D / 2;
    // LDS of a wavefront: d = 32, the P, Q and dO tiles and 64 floats of -g; d = 64, the P tile and two tiles each for
    // Q and dO, 20 KB, which eight wavefronts per CU fill to the last byte: -g then travels in a register, and the
    // buffer of the final reductions lies inside the tile space (CARVE), a barrier in between.
    constexpr bool CARVE = D == 64;
    constexpr int WB = D == 32 ? 3 * DmaTileF32::TILE + 256 : 5 * DmaTileF32::TILE;
    constexpr int RED = WAVES > 1 ? WAVES * (D / 32) * 16 * 64 * 4 : 0;
    static_assert(!CARVE || RED <= WAVES * WB, "the reduction fits in the tile space");
    __shared__ __attribute__((aligned(16))) char smem[CARVE ? WAVES * WB : WAVES * WB + (RED ? RED : 4)];
    float* lds = reinterpret_cast<float*>(CARVE ? smem : smem + WAVES * WB);
    const int item = xcd_remap(blockIdx.x, ns * NB);  // strips s0 .. s0+ns-1 of every head's strip order
    int bh, pos;
    item_to_head_strip(item, ns, hc, bh, pos);
    const int4 sd = reinterpret_cast<const int4*>(cdesc)[s0 + pos];  // strips longest first: {strip, first tile, tiles, 0}
    const int J = sd.x, e0 = sd.y, cnt = sd.z;
    const int w = wave_index(), l = threadIdx.x & 63, h = l >> 5, li = l & 31;
    size_t ib, ob, gb, hbytes, obytes, gbytes;
    int ild, old_, gld;
    head_slice<ST, D>(ly.in, ly.H, bh, L, ib, ild, hbytes);
    head_slice<ST, D>(ly.out, ly.H, bh, L, ob, old_, obytes);
    head_slice<ST, D>(ly.grad, ly.H, bh, L, gb, gld, gbytes);
    const rsrc_t rQ = make_rsrc(Q + ib, hbytes), rV = make_rsrc(Vt + ib, hbytes), rdO = make_rsrc(dO + ob, obytes);
    const rsrc_t rP = make_rsrc(P + (size_t)bh * nnz, (size_t)nnz * 4);
    const rsrc_t rG = make_rsrc(G + (size_t)bh * L, (size_t)L * 4);
    const int b_voff = (4 * h * ild + li) * 4, bo_voff = (4 * h * old_ + li) * 4;
    const int r_voff = (li * ild + h * KH) * 4, ro_voff = (li * old_ + h * KH) * 4;

    float vt[KH];
    if constexpr (VROW) ldr_rows<D>(rV, r_voff, J * 32 * ild * 4, vt);
    else ldr_cols<D>(rV, L, (h * KH * L + li) * 4, J * 128, vt);

    f32x16 ak[D / 32], av[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c) {
        ak[c] = splat16(0.f);
        av[c] = splat16(0.f);
    }
    // Per tile of the transposed index: {block row I, offset of the tile in this head's P, row stride}.
    const int4* __restrict__ desc = reinterpret_cast<const int4*>(tcdesc) + e0;
    const int nu = cnt > w ? (cnt - w + WAVES - 1) / WAVES : 0;  // tiles of this wavefront
    float* T = reinterpret_cast<float*>(smem + w * WB);
    if constexpr (D == 32) {
        // The P, Q and dO tiles and the 32 values of -g go straight into wave-private LDS (thirteen instructions, no
        // registers in flight); the operands of tile i are read out of LDS into registers -- the dO tile in both
        // of its roles -- then the same space is requested for tile i + 1, whose loads have the three chains of
        // tile i to arrive.
        const char* Tp = reinterpret_cast<const char*>(T);
        const char* Tq = Tp + DmaTileF32::TILE;
        const char* To = Tp + 2 * DmaTileF32::TILE;
        const char* Tg = Tp + 3 * DmaTileF32::TILE;
        const unsigned lp = lds_address(Tp), lq = lp + DmaTileF32::TILE, lo = lp + 2 * DmaTileF32::TILE,
                       lg = lp + 3 * DmaTileF32::TILE;
        const u32x4 wQ = rsrc_words(Q + ib, hbytes), wO = rsrc_words(dO + ob, obytes);
        const u32x4 wP = rsrc_words(P + (size_t)bh * nnz, (size_t)nnz * 4), wG = rsrc_words(G + (size_t)bh * L, (size_t)L * 4);
        const int ql = DmaTileF32::voff(l, ild), ol = DmaTileF32::voff(l, old_);
        const int qx = DmaTileF32::extra_step(ild), ox = DmaTileF32::extra_step(old_);
        const int pl0 = 16 * ((l & 7) ^ (l >> 3)), pl1 = (l >> 3) * 4;  // lane offset into a P tile: pl0 + pl1 * row stride
        const auto a_p = DmaTileF32::cols_addr(Tp, li, h), a_q = DmaTileF32::cols_addr(Tq, li, h),
                   a_o = DmaTileF32::cols_addr(To, li, h);
        const auto a_go = DmaTileF32::own_addr(To, li, 4 * h, 1);
        const char* a_g = Tg + 16 * h;
        auto issue = [&](const int4 d) {
            const int I = d.x, rn = d.z;
            DmaTileF32::load<true>(wP, lp, pl0 + pl1 * rn, d.y * 4, DmaTileF32::extra_step(rn));
            DmaTileF32::load(wQ, lq, ql, I * 32 * ild * 4, qx);
            DmaTileF32::load(wO, lo, ol, I * 32 * old_ * 4, ox);
            dma_b32(wG, lg, l * 4, I * 128);
        };
        settle(vt);
        if (nu > 0) {
            issue(desc[w]);
            int4 dn = desc[w + (nu > 1 ? WAVES : 0)];
            for (int i = 0; i < nu; ++i) {
                const int4 dnn = desc[w + min(i + 2, nu - 1) * WAVES];  // descriptor of the tile after the next
                wait_vm<0>();
                float pc[16], qb[1][16], ob[1][16], go[KH];
                f32x16 init;
                DmaTileF32::get(a_o, ob[0]);
                DmaTileF32::get(a_go, go);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x4 v = *reinterpret_cast<const f32x4*>(a_g + 32 * g);
                    init[4 * g + 0] = v.x;
                    init[4 * g + 1] = v.y;
                    init[4 * g + 2] = v.z;
                    init[4 * g + 3] = v.w;
                }
                DmaTileF32::get(a_p, pc);
                DmaTileF32::get(a_q, qb[0]);
                wait_lgkm0();
                if (i + 1 < nu) issue(dn);
                dn = dnn;
                __builtin_amdgcn_sched_barrier(0);
                f32x16 dp = mma_feat_init<D>(go, vt, init);  // dO_i . v_j - g_i, i = I*32+acc_row(r,h), j = J*32+li
                float ds[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) ds[r] = dp[r] * pc[r];
                mma_b<D>(ds, qb, ak);
                mma_b<D>(pc, ob, av);
            }
        }
    } else {
        // d = 64, the same schedule: the Q and dO tiles are two 4 KB tiles each (features 0..31 and 32..63), the P
        // tile one; twenty instructions a tile.  No room is left for -g: each lane loads the value of query row
        // lane % 32 of the next tile with an ordinary load (the compiler's wait for it falls where everything in
        // flight is waited for anyway, see settle), and one extra MFMA step -- A = that value in the lower half-wave,
        // zero in the upper, B = 1 -- spreads it over the accumulator the dP chain starts from.
        static_assert(D == 64, "head dimension 32 or 64");
        const char* Tp = reinterpret_cast<const char*>(T);
        const char* Tq = Tp + DmaTileF32::TILE;
        const char* To = Tp + 3 * DmaTileF32::TILE;
        const unsigned lp = lds_address(Tp), lq = lp + DmaTileF32::TILE, lo = lp + 3 * DmaTileF32::TILE;
        const u32x4 wQ = rsrc_words(Q + ib, hbytes), wO = rsrc_words(dO + ob, obytes);
        const u32x4 wP = rsrc_words(P + (size_t)bh * nnz, (size_t)nnz * 4);
        const int ql = DmaTileF32::voff(l, ild), ol = DmaTileF32::voff(l, old_);
        const int qx = DmaTileF32::extra_step(ild), ox = DmaTileF32::extra_step(old_);
        const int pl0 = 16 * ((l & 7) ^ (l >> 3)), pl1 = (l >> 3) * 4;  // lane offset into a P tile: pl0 + pl1 * row stride
        const auto a_p = DmaTileF32::cols_addr(Tp, li, h), a_q = DmaTileF32::cols_addr(Tq, li, h),
                   a_o = DmaTileF32::cols_addr(To, li, h);
        const auto a_go = DmaTileF32::own8_addr(To + h * DmaTileF32::TILE, li);  // dO[query li][feature 32h + s]
        auto issue = [&](const int4 d) {
            const int I = d.x, rn = d.z;
            DmaTileF32::load<true>(wP, lp, pl0 + pl1 * rn, d.y * 4, DmaTileF32::extra_step(rn));
            DmaTileF32::load(wQ, lq, ql, I * 32 * ild * 4, qx);
            DmaTileF32::load(wQ, lq + DmaTileF32::TILE, ql, I * 32 * ild * 4 + 128, qx);
            DmaTileF32::load(wO, lo, ol, I * 32 * old_ * 4, ox);
            DmaTileF32::load(wO, lo + DmaTileF32::TILE, ol, I * 32 * old_ * 4 + 128, ox);
        };
        settle(vt);
        if (nu > 0) {
            int4 dn = desc[w];
            issue(dn);
            float gl = ld1(rG, li * 4, dn.x * 128);
            dn = desc[w + (nu > 1 ? WAVES : 0)];
            for (int i = 0; i < nu; ++i) {
                const int4 dnn = desc[w + min(i + 2, nu - 1) * WAVES];  // descriptor of the tile after the next
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
                    issue(dn);
                    gl = ld1(rG, li * 4, dn.x * 128);
                }
                dn = dnn;
                __builtin_amdgcn_sched_barrier(0);
                const f32x16 init = __builtin_amdgcn_mfma_f32_32x32x2f32(ga, 1.0f, splat16(0.f), 0, 0, 0);  // -g_i in every column
                f32x16 dp = mma_feat_init<D>(go, vt, init);  // dO_i . v_j - g_i, i = I*32+acc_row(r,h), j = J*32+li
                float ds[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) ds[r] = dp[r] * pc[r];
                mma_b<D>(ds, qb, ak);
                mma_b<D>(pc, ob, av);
            }
        }
    }
    if constexpr (CARVE && WAVES > 1) __syncthreads();  // every wavefront is done with its tiles
#pragma unroll
    for (int c = 0; c < D / 32; ++c) ak[c] *= scale;
    reduce_store<D, WAVES>(ak, dK + gb, J * 32, w, li, h, lds, gld);
    if (WAVES > 1) __syncthreads();
    reduce_store<D, WAVES>(av, dV + gb, J * 32, w, li, h, lds, gld);
}

}  // namespace spion
