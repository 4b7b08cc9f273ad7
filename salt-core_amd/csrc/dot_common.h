// Pieces shared by the two tolerance-class decode kernels (affine Q4: q4_dot.hip, NVFP4: nvfp4_dot.hip): a wave owns a
// block of 32 rows and walks it in two strips, 128 bytes of each strip and row per step, 8 KiB per step fetched
// straight into LDS; the pieces below are the geometry constants, the compile-time step loop and the two kinds of
// wait.
#pragma once

#include "mi355_internal.h"

#ifndef DOT_SWIZZLE_LOW
#define DOT_SWIZZLE_LOW 0
#endif

#include <stddef.h>
#include <stdlib.h>

#include <type_traits>
#include <utility>

namespace mi355 {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef const u32x4 __attribute__((address_space(1))) *global_u128_ptr;
typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef const uint64_t __attribute__((address_space(4))) *uniform_u64_ptr;

constexpr int BLOCK_ROWS = DOT_BLOCK_ROWS;   // rows per block = N of the matrix instruction
constexpr int STAGE_BYTES = 8192;            // 2 strips x 32 rows x 128 bytes
constexpr int STAGE_GROUPS = 4;              // scale groups per strip and step
constexpr int STEP_LDS = STAGE_BYTES;
constexpr int LOADS_PER_STEP = 8;            // weight pieces
#ifndef DOT_STREAMING
#define DOT_STREAMING 2
#endif
constexpr int STREAMING = DOT_STREAMING;     // 2 = non-temporal: every weight byte is read once

__device__ __forceinline__ int swizzle(int piece) { return DOT_SWIZZLE_LOW ? (piece & 7) : ((piece >> 1) & 7); }

// steps per strip: half of the row's groups, in whole steps
__host__ __device__ __forceinline__ int dot_steps(int ngrp) { return ((ngrp + 1) / 2 + STAGE_GROUPS - 1) / STAGE_GROUPS; }

// f(integral_constant<int, 0>), f(<1>), ... until one returns false; true when all ran
template <int... I, class F>
__device__ __forceinline__ bool static_steps(std::integer_sequence<int, I...>, F &&f) {
    return (f(std::integral_constant<int, I>{}) && ...);
}

// A lane's scales (or biases) of one block: MD dwords = 2 * MD groups of its strip, in registers.
template <int MD> struct MetaRegs { u32x4 q[MD / 4]; };

// Written in assembly so that the compiler neither moves the load nor waits for it on its own: the one wait that
// covers it names the registers (wait_meta).
__device__ __forceinline__ u32x4 load_meta16(const uint8_t *address) {
    u32x4 value;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(value) : "v"(address) : "memory");
    return value;
}
__device__ __forceinline__ void wait_meta(u32x4 &value) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(value) : : "memory"); }

template <int N>
__device__ __forceinline__ void wait_vm() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

}  // namespace
}  // namespace mi355
