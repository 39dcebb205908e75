// Shared device helpers for the gfx950 W4A16 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace w4a16 {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kGroup = 128;

// AWQ order: bit position 4*i of a word holds natural column kPackOrder[i] of its block.
__host__ __device__ constexpr int pack_order(int i) { return ((i & 3) << 1) | (i >> 2); }      // 0,2,4,6,1,3,5,7
// Bit-position index that holds natural column j.
__host__ __device__ constexpr int unpack_pos(int j) { return ((j & 1) << 2) | (j >> 1); }      // 0,4,1,5,2,6,3,7

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) {
    return __builtin_bit_cast(float, bits16 << 16);
}

// Two fp32 -> packed bf16 pair (round-to-nearest-even, v_cvt_pk_bf16_f32): low half = a.
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    bf16x2 v;
    v.x = static_cast<__bf16>(a);
    v.y = static_cast<__bf16>(b);
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ uint16_t float_to_bf16_bits(float a) {
    __bf16 v = static_cast<__bf16>(a);
    return __builtin_bit_cast(uint16_t, v);
}

// Nibble at bit-position index `pos` of `w` as float (exact).
__device__ __forceinline__ float nibble_f32(uint32_t w, int pos) {
    return static_cast<float>((w >> (4 * pos)) & 0xFu);
}

// The 8 nibbles of one AWQ word as floats in NATURAL column order.  The even/odd
// nibble split lets every conversion be a byte-select convert (v_cvt_f32_ubyteN).
__device__ __forceinline__ void unpack8_f32(uint32_t w, float (&q)[8]) {
    const uint32_t e = w & 0x0F0F0F0Fu;          // positions 0,2,4,6 -> columns 0,4,1,5
    const uint32_t o = (w >> 4) & 0x0F0F0F0Fu;   // positions 1,3,5,7 -> columns 2,6,3,7
    q[0] = static_cast<float>(e & 0xFFu);
    q[4] = static_cast<float>((e >> 8) & 0xFFu);
    q[1] = static_cast<float>((e >> 16) & 0xFFu);
    q[5] = static_cast<float>(e >> 24);
    q[2] = static_cast<float>(o & 0xFFu);
    q[6] = static_cast<float>((o >> 8) & 0xFFu);
    q[3] = static_cast<float>((o >> 16) & 0xFFu);
    q[7] = static_cast<float>(o >> 24);
}

// Maximum / sum over the 64 lanes of a wavefront, every lane receiving the result: the four steps inside a row of
// 16 lanes on DPP moves (quad permutes for distances 1 and 2, half-row and row mirrors for 4 and 8: once the
// quads agree, mirroring meets the partner quad), the two steps across rows by shuffle.
template <bool MAX>
__device__ __forceinline__ float wave_reduce(float v) {
    auto op = [](float a, float b) { return MAX ? fmaxf(a, b) : a + b; };
    auto dpp = [&](auto ctrl) {
        constexpr int CTRL = decltype(ctrl)::value;
        const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
        v = op(v, __builtin_bit_cast(float, moved));
    };
    dpp(std::integral_constant<int, 0xB1>());    // quad_perm [1, 0, 3, 2]
    dpp(std::integral_constant<int, 0x4E>());    // quad_perm [2, 3, 0, 1]
    dpp(std::integral_constant<int, 0x141>());   // row_half_mirror
    dpp(std::integral_constant<int, 0x140>());   // row_mirror
    v = op(v, __shfl_xor(v, 16));
    return op(v, __shfl_xor(v, 32));
}

// Sum over the 16 lanes of a DPP row, every lane of the row receiving it (the four in-row steps of wave_reduce).
__device__ __forceinline__ float row_sum16(float v) {
    auto dpp = [&](auto ctrl) {
        constexpr int CTRL = decltype(ctrl)::value;
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
    };
    dpp(std::integral_constant<int, 0xB1>());    // quad_perm [1, 0, 3, 2]
    dpp(std::integral_constant<int, 0x4E>());    // quad_perm [2, 3, 0, 1]
    dpp(std::integral_constant<int, 0x141>());   // row_half_mirror
    dpp(std::integral_constant<int, 0x140>());   // row_mirror
    return v;
}

// silu(g) in the reference's tanh form (matvec_int4_swiglu_rms.py:512-514), fp32
__device__ __forceinline__ float silu_tanh(float g) { return g * 0.5f * (tanhf(g * 0.5f) + 1.0f); }

// "No score yet" of the attention partials: finite, so differences of two of them are 0, not NaN.
constexpr float kAttnNegBig = -1e30f;

// Agent-scope (all XCDs) relaxed accesses for data exchanged between workgroups.
__device__ __forceinline__ void store_agent(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace w4a16
