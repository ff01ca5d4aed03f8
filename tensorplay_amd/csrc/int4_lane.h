// Per-lane helpers shared by the int4 decode kernels: nibble -> 16-bit float
// conversion in place, v_dot2 / MFMA wrappers, for fp16 and bf16 activations.
#pragma once

#include "tpq_common.h"

namespace tpq {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef short short2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t word2_t __attribute__((ext_vector_type(2)));

constexpr int kDecodeWaves = 16;  // 1024 threads: the whole K range of 64 columns in one workgroup
constexpr int kChunkKT = 4;       // k-tiles (of 32) per chunk
constexpr int kRing = 2;          // chunks in flight per wavefront

// (a & mask) | magic, meant to become one v_and_or_b32.  That instruction takes a single
// scalar operand on this target, so callers keep `magic` in a VGPR (loaded through an opaque
// v_mov) and the mask sits in an SGPR.
//
// FOR_MFMA = true: plain C, because the compiler has to see the instruction to insert the wait
// states a following MFMA needs (an inline-assembly result fed straight into an MFMA read
// garbage).  FOR_MFMA = false (result consumed by ordinary VALU ops such as v_dot2): the
// instruction is spelled out, which keeps the compiler from adding a register move per use.
template <bool FOR_MFMA>
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
    if constexpr (FOR_MFMA) {
        return (a & mask) | magic;
    } else {
        uint32_t r;
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
        return r;
    }
}

template <int DT>
struct Lane16;

template <>
struct Lane16<TPQ_DTYPE_F16> {
    // pairs j = 0, 2 sit in bits 0..3 / 16..19 (of w, w >> 8): exponent 0x6400 makes them 1024 + c;
    // pairs j = 1, 3 sit in bits 4..7 / 20..23: exponent 0x5400 makes them 64 + c.
    static constexpr float kOffsetEven = 1032.0f, kOffsetOdd = 72.0f;  // magic + 8 (code bias)
    static constexpr bool kUseMfma = true;
    static constexpr uint32_t kMagicEven = 0x64006400u, kMagicOdd = 0x54005400u, kOnes = 0x3C003C00u;
    static __device__ __forceinline__ float dot(uint32_t x, uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, x), __builtin_bit_cast(half2_t, w), acc, false);
    }
    // v_mfma_f32_4x4x4_16B_f16: 16 independent 4x4x4 products; a/b are two words = four k each
    static __device__ __forceinline__ float4_t mfma(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
        const word2_t a = {a0, a1}, b = {b0, b1};
        return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, a), __builtin_bit_cast(half4_t, b), c, 0, 0, 0);
    }
    template <bool FOR_MFMA>
    static __device__ __forceinline__ void unpack(uint32_t w, uint32_t (&v)[4], uint32_t magic_even, uint32_t magic_odd) {
        const uint32_t w8 = w >> 8;
        v[0] = and_or<FOR_MFMA>(w, 0x000F000Fu, magic_even);
        v[1] = and_or<FOR_MFMA>(w, 0x00F000F0u, magic_odd);
        v[2] = and_or<FOR_MFMA>(w8, 0x000F000Fu, magic_even);
        v[3] = and_or<FOR_MFMA>(w8, 0x00F000F0u, magic_odd);
    }
    static __device__ __forceinline__ float lo(uint32_t p) { return f16_bits_to_f32(p & 0xFFFFu); }
    static __device__ __forceinline__ float hi(uint32_t p) { return f16_bits_to_f32(p >> 16); }
    static __device__ __forceinline__ uint16_t out(float v) { return f32_to_f16_bits(v); }
};

template <>
struct Lane16<TPQ_DTYPE_BF16> {
    // bf16 has 7 mantissa bits: a nibble only fits in bits 0..3, so every pair is shifted down
    // and becomes 128 + c.
    static constexpr float kOffsetEven = 136.0f, kOffsetOdd = 136.0f;
    static constexpr bool kUseMfma = false;  // the streaming kernel keeps v_dot2_f32_bf16 for bf16
    static constexpr uint32_t kMagicEven = 0x43004300u, kMagicOdd = 0x43004300u, kOnes = 0x3F803F80u;
    static __device__ __forceinline__ float dot(uint32_t x, uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(short2_t, x), __builtin_bit_cast(short2_t, w), acc, false);
    }
    static __device__ __forceinline__ float4_t mfma(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
        const word2_t a = {a0, a1}, b = {b0, b1};
        return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
    }
    template <bool FOR_MFMA>
    static __device__ __forceinline__ void unpack(uint32_t w, uint32_t (&v)[4], uint32_t magic_even, uint32_t) {
        v[0] = and_or<FOR_MFMA>(w, 0x000F000Fu, magic_even);
        v[1] = and_or<FOR_MFMA>(w >> 4, 0x000F000Fu, magic_even);
        v[2] = and_or<FOR_MFMA>(w >> 8, 0x000F000Fu, magic_even);
        v[3] = and_or<FOR_MFMA>(w >> 12, 0x000F000Fu, magic_even);
    }
    static __device__ __forceinline__ float lo(uint32_t p) { return bf16_bits_to_f32(p & 0xFFFFu); }
    static __device__ __forceinline__ float hi(uint32_t p) { return bf16_bits_to_f32(p >> 16); }
    static __device__ __forceinline__ uint16_t out(float v) { return f32_to_bf16_bits(v); }
};

}  // namespace
}  // namespace tpq
