// Shared device helpers for the gfx950 block-sparse kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pbs {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct bf16_t {
    uint16_t bits;
};

// Per element type: bytes, and how one 32x32x32 block product is issued on the matrix cores.
//
// A "fragment" is what one lane holds of a 32(rows) x 32(k) operand tile: lane l serves row
// (l & 31) and the 16 consecutive k values 16*(l >> 5) .. +15, kept as NQ 16-byte registers
// quads.  Both operands of a product use the same assignment of k to (lane half, register),
// so any operand whose k runs contiguously in memory is loaded with plain 16-byte reads.
template <typename T>
struct Elem;

template <>
struct Elem<float> {
    static constexpr int ESZ = 4;
    static constexpr int NQ = 4;  // 16 floats per lane
    // v_mfma_f32_32x32x2_f32: lane half h supplies k = h of each 2-wide step; here step
    // (q, e) contracts the k pair {4q+e, 16+4q+e}.
    static __device__ __forceinline__ void mma(f32x16& acc, const uint4* a, const uint4* b) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[q].x), __uint_as_float(b[q].x), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[q].y), __uint_as_float(b[q].y), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[q].z), __uint_as_float(b[q].z), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[q].w), __uint_as_float(b[q].w), acc, 0, 0, 0);
        }
    }
    static __device__ __forceinline__ float from_f32(float v) { return v; }
    static __device__ __forceinline__ float to_f32(float v) { return v; }
};

template <>
struct Elem<bf16_t> {
    static constexpr int ESZ = 2;
    static constexpr int NQ = 2;  // 16 bf16 per lane
    // v_mfma_f32_32x32x16_bf16: lane half h supplies 8 consecutive k of each 16-wide step;
    // here step q contracts k in {8q..8q+7} u {16+8q..16+8q+7}.
    static __device__ __forceinline__ void mma(f32x16& acc, const uint4* a, const uint4* b) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[q]),
                                                          __builtin_bit_cast(bf16x8, b[q]), acc, 0, 0, 0);
        }
    }
    // round to nearest even, NaN kept quiet: the hardware conversion (v_cvt_pk_bf16_f32, two values per
    // instruction where the compiler can pair them)
    static __device__ __forceinline__ bf16_t from_f32(float v) {
        bf16_t r;
        r.bits = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
        return r;
    }
    static __device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }
};

// Row of accumulator register v (0..15) held by a lane of half h in a 32x32 MFMA result;
// the column is (lane & 31).
static __device__ __forceinline__ int acc_row(int v, int h) { return 8 * (v >> 2) + 4 * h + (v & 3); }

// A row/column pointer value read from a caller's index array, forced into [0, nnz]: a corrupt
// pointer array then selects wrong entries instead of reading outside the entry list.
static __device__ __forceinline__ int clamp_entry(int v, int nnz) { return v < 0 ? 0 : (v > nnz ? nnz : v); }

static __device__ __forceinline__ uint4 ldg16(const void* p) { return *reinterpret_cast<const uint4*>(p); }

// Two 16-byte rows of 8 bf16 (row k even, row k odd, same 8 columns) -> 8 words, word n holding
// (row_even[n] low half, row_odd[n] high half): the k-pair packing the bf16 MFMA operands want.
static __device__ __forceinline__ void interleave_bf16_rows(const uint4& r0, const uint4& r1, uint4& lo, uint4& hi) {
    lo.x = (r0.x & 0xffffu) | (r1.x << 16);
    lo.y = (r0.x >> 16) | (r1.x & 0xffff0000u);
    lo.z = (r0.y & 0xffffu) | (r1.y << 16);
    lo.w = (r0.y >> 16) | (r1.y & 0xffff0000u);
    hi.x = (r0.z & 0xffffu) | (r1.z << 16);
    hi.y = (r0.z >> 16) | (r1.z & 0xffff0000u);
    hi.z = (r0.w & 0xffffu) | (r1.w << 16);
    hi.w = (r0.w >> 16) | (r1.w & 0xffff0000u);
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lane s passes the LDS address of 4 consecutive
// 16-bit elements (row s/4 of a 4 x 16 tile, columns 4*(s%4)..+3) and lane j receives column j of
// the tile: the 4 rows' elements, in row order.
static __device__ __forceinline__ uint2 tr16_b64(const unsigned char* lds_ptr) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(lds_ptr));
    return __builtin_bit_cast(uint2, v);
}

// Volatile accesses to LDS words other waves write or poll.  The pointer is cast to the LDS address
// space explicitly: a volatile access through a generic pointer is compiled to a flat instruction,
// which takes the long way round through the vector memory path.
typedef int __attribute__((address_space(3))) lds_int;
static __device__ __forceinline__ int lds_peek(const int* p) { return *(const volatile lds_int*)p; }
static __device__ __forceinline__ void lds_poke(int* p, int v) { *(volatile lds_int*)p = v; }

// Waits of the barrier-free kernels that ran into their bound, counted over the life of the process (one word per
// GPU).  Such a wait means a broken progress protocol; the kernel also turns the affected results into NaN.
static __device__ unsigned g_protocol_failures;
static __device__ __forceinline__ void count_protocol_failure() {
    if ((threadIdx.x & 63) == 0) atomicAdd(&g_protocol_failures, 1u);
}

// a wave-uniform pointer, forced into scalar registers
static __device__ __forceinline__ const unsigned char* uniform_ptr(const unsigned char* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const unsigned char*>(((uint64_t)hi << 32) | lo);
}

// one DMA instruction: lane p copies the 16 bytes at base + voff to LDS chunk (lds_base/16 + p).
// M0 is written inside the statement and cannot be named as a clobber (the compiler treats it as a
// reserved register and rejects that with a warning about undefined behaviour); these kernels contain
// nothing else that makes the compiler use M0 (no LDS-DMA builtins, no dynamically indexed registers).
static __device__ __forceinline__ void dma16(unsigned lds_base_uniform, const unsigned char* base_uniform, unsigned voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t"
                 :
                 : "s"(lds_base_uniform), "v"(voff), "s"(base_uniform)
                 : "memory");
}

// wait until at most n (wave-uniform) of this wave's DMA loads are outstanding, make this wave's
// LDS accesses complete, and meet the other waves.  Loads retire in order, so a smaller n than
// necessary is only slower, never wrong.
static __device__ __forceinline__ void wait_dma_and_barrier(int n) {
#define PBS_W(N) case N: asm volatile("s_waitcnt vmcnt(" #N ") lgkmcnt(0)\n\ts_barrier" ::: "memory"); break;
    switch (n) {
        PBS_W(0) PBS_W(1) PBS_W(2) PBS_W(3) PBS_W(4) PBS_W(5) PBS_W(6) PBS_W(7) PBS_W(8)
        PBS_W(9) PBS_W(10) PBS_W(11) PBS_W(12) PBS_W(13) PBS_W(14) PBS_W(15) PBS_W(16)
        PBS_W(17) PBS_W(18) PBS_W(19) PBS_W(20) PBS_W(21) PBS_W(22) PBS_W(23) PBS_W(24)
        PBS_W(25) PBS_W(26) PBS_W(27) PBS_W(28) PBS_W(29) PBS_W(30) PBS_W(31) PBS_W(32)
        PBS_W(33) PBS_W(34) PBS_W(35) PBS_W(36) PBS_W(37) PBS_W(38) PBS_W(39) PBS_W(40)
        PBS_W(41) PBS_W(42) PBS_W(43) PBS_W(44) PBS_W(45) PBS_W(46) PBS_W(47) PBS_W(48)
        default: asm volatile("s_waitcnt vmcnt(48) lgkmcnt(0)\n\ts_barrier" ::: "memory"); break;
    }
#undef PBS_W
}
// the 4-byte form: lane p copies the 4 bytes at base + voff to LDS word (lds_base/4 + p)
static __device__ __forceinline__ void dma4(unsigned lds_base_uniform, const unsigned char* base_uniform, unsigned voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n\t"
                 :
                 : "s"(lds_base_uniform), "v"(voff), "s"(base_uniform)
                 : "memory");
}

// wait until at most n (wave-uniform) of this wave's DMA loads are outstanding
static __device__ __forceinline__ void wait_dma(int n) {
#define PBS_W(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    switch (n) {
        PBS_W(0) PBS_W(1) PBS_W(2) PBS_W(3) PBS_W(4) PBS_W(5) PBS_W(6) PBS_W(7) PBS_W(8)
        PBS_W(9) PBS_W(10) PBS_W(11) PBS_W(12) PBS_W(13) PBS_W(14) PBS_W(15) PBS_W(16)
        PBS_W(17) PBS_W(18) PBS_W(19) PBS_W(20) PBS_W(21) PBS_W(22) PBS_W(23) PBS_W(24)
        PBS_W(25) PBS_W(26) PBS_W(27) PBS_W(28) PBS_W(29) PBS_W(30) PBS_W(31) PBS_W(32)
        PBS_W(33) PBS_W(34) PBS_W(35) PBS_W(36) PBS_W(37) PBS_W(38) PBS_W(39) PBS_W(40)
        PBS_W(41) PBS_W(42) PBS_W(43) PBS_W(44) PBS_W(45) PBS_W(46) PBS_W(47) PBS_W(48)
        default: asm volatile("s_waitcnt vmcnt(48)" ::: "memory"); break;
    }
#undef PBS_W
}
// barrier of a wave that has no DMA in flight or does not care (its LDS accesses complete first)
static __device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
static __device__ __forceinline__ void drain_barrier() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

static constexpr int NUM_XCD = 8;

// Workgroups are handed to the 8 XCDs round-robin by id.  Give each XCD one contiguous range of
// logical tile ids, walked in launch order, so tiles that share an operand panel run on the same
// XCD (one L2) at about the same time.  Returns -1 for the padding ids of the last range.
static __device__ __forceinline__ int xcd_tile_id(int wg, int total) {
    const int per = (total + NUM_XCD - 1) / NUM_XCD;
    const int id = (wg % NUM_XCD) * per + wg / NUM_XCD;
    return id < total ? id : -1;
}
static inline int xcd_grid(int total) { return ((total + NUM_XCD - 1) / NUM_XCD) * NUM_XCD; }

}  // namespace pbs
