// Building blocks shared by the kernels that keep a (32 headdim rows) x (all dstate columns) state tile per wave
// (gfx950): register types, bf16 packing, buffer descriptors, explicit wait-count immediates, and the 16-byte
// state store with its data hazard guard.
#pragma once
#include "ssd_params.h"

#include <utility>

namespace ssd {
namespace tile {

// compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{})
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) { static_for_impl(std::make_integer_sequence<int, N>{}, f); }

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, int64_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)(bytes > 0x7fffffffLL ? 0x7fffffffLL : (bytes < 0 ? 0 : bytes)),
                                             0x00020000);
}

// s_waitcnt immediate that only waits for the vector-memory counter to drop to n (gfx9 field layout)
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }

// Four consecutive fp32 state values of one row.  The data registers of a wide store are read out over several
// cycles after issue; wait states that depend on them keep a following writer of the same registers away.
// aux: cache policy bits of the store (0 = default; 1 = sc0, 2 = nt, 16 = sc1).
__device__ __forceinline__ void store4_f32(__amdgpu_buffer_rsrc_t rs, int voff, int soff, f32x4 v, int aux = 0)
{
    const u32x4 q = __builtin_bit_cast(u32x4, v);
    if (aux == 17) __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 17);
    else if (aux == 16) __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 16);
    else if (aux == 1) __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 1);
    else __builtin_amdgcn_raw_buffer_store_b128(q, rs, 4 * voff, 4 * soff, 0);
    asm volatile("s_nop 3" ::"v"(q) : "memory");
}

// bf16 hi / lo halves of the scaled x operand of one 32-token step: [row parity][token pair]
struct Frag { uint32_t hi[2][4], lo[2][4]; };

}  // namespace tile
}  // namespace ssd
