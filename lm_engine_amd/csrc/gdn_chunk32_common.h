// Device helpers shared by the kernels built on v_mfma_f32_32x32x16_bf16 (gdn_chunk32.hip, gdn_chunk_fused.hip).
#pragma once

#include <type_traits>

#include "gdn_chunk_common.h"

namespace gdn {

typedef __attribute__((ext_vector_type(4))) short s16x4;

__device__ __forceinline__ bf16x8 pack8_16(const f32x16& d, int s, float sign) {
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; e++) r[e] = (bf16_t)(sign * d[8 * s + e]);
    return r;
}

// 4 consecutive rows x 16 consecutive columns of a row-major bf16 LDS matrix, transposed on the
// way in: lane i of each 16-lane group receives M[row0 + 0..3][col0 + i].
// With SWAP, the two middle groups of 4 columns change places: lane i receives column col0 + sigma(i),
// sigma(4 q + b) = 4 swap(q) + b, swap(1) = 2, swap(2) = 1 (the column order of the scan's state slices).
template <bool SWAP = false>
__device__ __forceinline__ bf16x4 lds_read_tr4x16(const bf16_t* m, int ld, int row0, int col0, int l16) {
    const int q = l16 % 4;
    const int piece = SWAP ? ((q & 1) << 1 | (q >> 1)) : q;
    const bf16_t* p = m + (row0 + l16 / 4) * ld + col0 + 4 * piece;
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
    return __builtin_bit_cast(bf16x4, v);
}

// Column of a 32-column state slice held by lane l32 (the order lds_read_tr4x16<true> produces): with it,
// register pair (2 m, 2 m + 1) of a transposed accumulator tile covers 8 consecutive columns per lane.
__device__ __forceinline__ int slice_col(int l32) { return (l32 & 0x13) | ((l32 & 4) << 1) | ((l32 & 8) >> 1); }

// compile-time loop: f(std::integral_constant<int, I>{}) for I = B .. E - 1
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// keeps the computation of x at this point of the program
__device__ __forceinline__ void pin_regs(bf16x8& x) {
    typedef __attribute__((ext_vector_type(4))) int i32x4;
    i32x4 t = __builtin_bit_cast(i32x4, x);
    asm volatile("" : "+v"(t));
    x = __builtin_bit_cast(bf16x8, t);
}

// ---- hand-over between two waves of a workgroup through LDS ----
// A wave publishes what it wrote to LDS by storing a running epoch number to an LDS word of its own; the other wave
// polls that word.  LDS operations of a wave execute in order, so whoever reads the new epoch reads the data written
// before it.  The words are addressed as LDS explicitly: through a generic pointer the compiler emits FLAT accesses,
// which take the vector-memory path and are not ordered with the DS instructions around them.
typedef __attribute__((address_space(3))) volatile int lds_flag_t;

__device__ __forceinline__ void pair_publish(lds_flag_t* flag, int epoch) {
    asm volatile("" ::: "memory");
    *flag = epoch;
    asm volatile("" ::: "memory");
}

// The wait is one asm statement, loop included, so that the chunk loop of a compute wave stays a single basic
// block: with a branch in it the compiler sinks work that is not needed until after the wait past it, out of the
// slots it was written into.  All lanes read the same word.
__device__ __forceinline__ void pair_wait(lds_flag_t* flag, int epoch) {
    int seen, uniform;
    asm volatile(
        "pair_wait_%=:\n\t"
        "ds_read_b32 %0, %2\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        "v_readfirstlane_b32 %1, %0\n\t"
        "s_cmp_lt_i32 %1, %3\n\t"
        "s_cbranch_scc1 pair_wait_%="
        : "=&v"(seen), "=&s"(uniform)
        : "v"((uint32_t)(uintptr_t)flag), "s"(epoch)
        : "memory", "scc");
}

}  // namespace gdn
