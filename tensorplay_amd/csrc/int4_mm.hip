// int4 group-quantized weight-only matmul for gfx950, decode shapes first.
//
//   y[m,n] = sum_k x[m,k] * ((code[n,k] - 8) * scale[k/g,n] + zero[k/g,n])
//
// Packed weight (written by tpq_int4_pack with innerKTiles = 2): int32
// [N/8][K/32][32] words.  Word t of tile (nT, kT) belongs to row
// n = 8 nT + t/4 and holds the eight codes at k = 32 kT + 2 (t%4) + 8 j + {0,1}:
// bits[4j..] are the even one, bits[16+4j..] the odd one.  The four words of a
// row (t%4 = 0..3) are adjacent, so 16 bytes = one row x 32 consecutive k.
//
// Decode kernel (M <= 4, fp16/bf16, K % 128 == 0), bandwidth bound:
//   * a workgroup owns 64 consecutive output columns; lane l of every
//     wavefront owns column 64*block + l, i.e. row l%8 of tile l/8, and reads
//     its 16 bytes per k-tile with one dwordx4 load (a wavefront reads eight
//     whole 128-byte lines, one per tile);
//   * the k range is dealt to the 16 wavefronts of the workgroup in chunks of
//     four k-tiles (128 k), so all lanes of a wavefront work on the SAME k
//     values: the activations are wave-uniform and are fetched with scalar
//     loads straight into SGPRs, which feed v_dot2_f32_f16 / v_dot2_f32_bf16
//     as the scalar operand - no LDS traffic and no cross-lane traffic for x;
//   * nibbles become 16-bit floats in place with the "magic exponent" trick:
//     ((w << 4) & 0x00F000F0) | 0x54005400 is the fp16 pair (64+c_even, 64+c_odd)
//     (bf16: (w & 0x000F000F) | 0x43004300 = 128 + c), one shift and one
//     v_and_or_b32 per pair;
//   * the offset is removed per group, not per element: with
//     p = sum x (OFF + c) and sx = sum x over the group,
//     y += scale * (p - (OFF + 8) * sx) + zero * sx, all in fp32.  sx comes
//     from one extra coalesced load of the chunk's 64 activation words (lane l
//     takes word l), a dot with (1,1) and a 16-lane butterfly;
//   * each wavefront keeps two chunks (128 bytes per lane) in flight;
//   * the wavefronts' partial columns meet in LDS and are stored once.
//
// Everything else (fp32 activations, other K, unaligned pointers) goes
// through a plain fp32 kernel that evaluates w = fma(code-8, scale, zero),
// y = fma(x, w, y) like the reference's CPU kernel
// (p10/src/backend/cpu/QuantizedElementwiseKernels.cpp:470-479).
#include "tpq_common.h"

namespace tpq {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef short short2_t __attribute__((ext_vector_type(2)));

constexpr int kDecodeWaves = 16;  // 1024 threads: the whole K range of 64 columns in one workgroup
constexpr int kChunkKT = 4;       // k-tiles (of 32) per chunk
constexpr int kRing = 2;          // chunks in flight per wavefront

// (a & mask) | magic in one VALU op; magic lives in a VGPR, mask in an SGPR
// (one constant-bus operand per instruction on this target).
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
    return r;
}

template <int DT>
struct Lane16;

template <>
struct Lane16<TPQ_DTYPE_F16> {
    static constexpr float kOffset = 72.0f;  // 64 (magic) + 8 (code bias)
    static constexpr uint32_t kMask = 0x00F000F0u, kMagic = 0x54005400u, kOnes = 0x3C003C00u;
    static __device__ __forceinline__ float dot(uint32_t x, uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, x), __builtin_bit_cast(half2_t, w), acc, false);
    }
    // pair j of word w (codes at k0 + 8j, k0 + 8j + 1) moved to bits 4..7 / 20..23
    static __device__ __forceinline__ uint32_t align(uint32_t w, int j) {
        return j == 0 ? (w << 4) : (j == 1 ? w : (w >> (4 * j - 4)));
    }
    static __device__ __forceinline__ float lo(uint32_t p) { return f16_bits_to_f32(p & 0xFFFFu); }
    static __device__ __forceinline__ float hi(uint32_t p) { return f16_bits_to_f32(p >> 16); }
    static __device__ __forceinline__ uint16_t out(float v) { return f32_to_f16_bits(v); }
};

template <>
struct Lane16<TPQ_DTYPE_BF16> {
    static constexpr float kOffset = 136.0f;  // 128 (magic) + 8
    static constexpr uint32_t kMask = 0x000F000Fu, kMagic = 0x43004300u, kOnes = 0x3F803F80u;
    static __device__ __forceinline__ float dot(uint32_t x, uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(short2_t, x), __builtin_bit_cast(short2_t, w), acc, false);
    }
    static __device__ __forceinline__ uint32_t align(uint32_t w, int j) { return j == 0 ? w : (w >> (4 * j)); }
    static __device__ __forceinline__ float lo(uint32_t p) { return bf16_bits_to_f32(p & 0xFFFFu); }
    static __device__ __forceinline__ float hi(uint32_t p) { return bf16_bits_to_f32(p >> 16); }
    static __device__ __forceinline__ uint16_t out(float v) { return f32_to_bf16_bits(v); }
};

// One chunk in flight: 4 k-tiles x 16 bytes of weights, the (scale, zero)
// words of its groups, and this lane's word of the chunk's activations.
template <int MROWS, int GROUPS>
struct Chunk {
    uint4 q[kChunkKT];
    uint32_t p[GROUPS];
    uint32_t xw[MROWS];
};

// x: [M][K/2] 32-bit words (pairs of 16-bit floats); sz: [G][N] words (scale, zero);
// GROUP_KT = group / 32 in {1, 2, 4}; k_super % 4 == 0.
template <int DT, int MROWS, int GROUP_KT>
__global__ __launch_bounds__(kDecodeWaves* kWave) void int4_decode_kernel(
    const uint32_t* __restrict__ x, const uint4* __restrict__ packed, const uint32_t* __restrict__ sz,
    uint16_t* __restrict__ y, int N, int K, int k_super) {
    using L = Lane16<DT>;
    constexpr int kGroups = kChunkKT / GROUP_KT;
    __shared__ float red[kDecodeWaves * MROWS * kWave];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = blockIdx.x * kWave + lane;
    const int n_ld = n < N ? n : N - 1;  // lanes past the edge read a valid column and drop the result
    const uint4* wp = packed + (static_cast<size_t>(n_ld >> 3) * k_super) * 8 + (n_ld & 7);
    const uint32_t* szp = sz + n_ld;
    const int words_per_row = K >> 1;
    const int n_chunks = k_super / kChunkKT;

    uint32_t magic;
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(L::kMagic));

    auto issue = [&](Chunk<MROWS, kGroups>& ch, int chunk) {
        chunk = chunk < n_chunks ? chunk : n_chunks - 1;  // past the end: harmless re-read, never used
#pragma unroll
        for (int i = 0; i < kChunkKT; ++i) ch.q[i] = wp[static_cast<size_t>(chunk * kChunkKT + i) * 8];
#pragma unroll
        for (int g = 0; g < kGroups; ++g) ch.p[g] = szp[static_cast<size_t>(chunk * kGroups + g) * N];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) ch.xw[m] = x[static_cast<size_t>(m) * words_per_row + chunk * 64 + lane];
    };

    float yacc[MROWS];
#pragma unroll
    for (int m = 0; m < MROWS; ++m) yacc[m] = 0.0f;

    auto consume = [&](const Chunk<MROWS, kGroups>& ch, int chunk) {
        // per k-tile sums of the activations: lanes 16i..16i+15 reduce k-tile i
        float xs[MROWS];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
            float s = L::dot(ch.xw[m], L::kOnes, 0.0f);
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) s += __shfl_xor(s, off, kWave);
            xs[m] = s;
        }
        float part[MROWS];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) part[m] = 0.0f;
#pragma unroll
        for (int i = 0; i < kChunkKT; ++i) {
            const int kt = __builtin_amdgcn_readfirstlane(chunk * kChunkKT + i);
            const uint32_t wq[4] = {ch.q[i].x, ch.q[i].y, ch.q[i].z, ch.q[i].w};
            uint32_t v[4][4];
#pragma unroll
            for (int t4 = 0; t4 < 4; ++t4)
#pragma unroll
                for (int j = 0; j < 4; ++j) v[t4][j] = and_or(L::align(wq[t4], j), L::kMask, magic);
#pragma unroll
            for (int m = 0; m < MROWS; ++m) {
                // wave-uniform address: scalar loads into SGPRs
                const uint32_t* xk = x + static_cast<size_t>(m) * words_per_row + kt * 16;
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int t4 = 0; t4 < 4; ++t4) part[m] = L::dot(xk[t4 + 4 * j], v[t4][j], part[m]);
                if (MROWS > 1) __builtin_amdgcn_sched_barrier(0);  // one row's activations in SGPRs at a time
            }
            if ((i + 1) % GROUP_KT == 0) {  // group boundary: fold the partial sums
                const uint32_t pw = ch.p[i / GROUP_KT];
                const float scale = L::lo(pw), zero = L::hi(pw);
#pragma unroll
                for (int m = 0; m < MROWS; ++m) {
                    float sx = 0.0f;
#pragma unroll
                    for (int g = 0; g < GROUP_KT; ++g)
                        sx += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xs[m]), 16 * (i + 1 - GROUP_KT + g)));
                    const float dotp = __builtin_fmaf(-L::kOffset, sx, part[m]);
                    yacc[m] = __builtin_fmaf(scale, dotp, yacc[m]);
                    yacc[m] = __builtin_fmaf(zero, sx, yacc[m]);
                    part[m] = 0.0f;
                }
            }
            // keep the k-tiles in program order: without this the scheduler unpacks
            // every tile of the chunk up front and runs out of registers
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    Chunk<MROWS, kGroups> ring[kRing];
#pragma unroll
    for (int u = 0; u < kRing; ++u) issue(ring[u], wave + u * kDecodeWaves);
    for (int c = wave; c < n_chunks; c += kRing * kDecodeWaves) {
#pragma unroll
        for (int u = 0; u < kRing; ++u) {
            const int cu = c + u * kDecodeWaves;
            if (cu < n_chunks) {
                consume(ring[u], cu);
                if (cu + kRing * kDecodeWaves < n_chunks) issue(ring[u], cu + kRing * kDecodeWaves);
            }
        }
    }

#pragma unroll
    for (int m = 0; m < MROWS; ++m) red[(wave * MROWS + m) * kWave + lane] = yacc[m];
    __syncthreads();
    if (tid < MROWS * kWave) {
        const int m = tid >> 6;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; ++w) s += red[(w * MROWS + m) * kWave + lane];
        if (n < N) y[static_cast<size_t>(m) * N + n] = L::out(s);
    }
}

// Plain fp32 evaluation for every case the decode kernel does not take.
// Workgroup = one tile of 8 columns x one activation row; thread t: row t%8,
// k-tiles t/8, t/8 + 32, ...
template <int DT>
__global__ __launch_bounds__(256) void int4_generic_kernel(
    const typename Elem<DT>::storage* __restrict__ x, const uint32_t* __restrict__ packed,
    const typename Elem<DT>::storage* __restrict__ sz, typename Elem<DT>::storage* __restrict__ y,
    int64_t N, int64_t K, int64_t k_super, int64_t group) {
    __shared__ float red[256];
    const int t = threadIdx.x, r = t & 7;
    const int64_t nT = blockIdx.x, m = blockIdx.y;
    const int64_t n = nT * 8 + r;
    const auto* xr = x + m * K;
    float acc = 0.0f;
    for (int64_t kt = t >> 3; kt < k_super; kt += 32) {
        const uint32_t* wq = packed + ((nT * k_super + kt) * 32 + r * 4);
        const int64_t g = (kt * 32) / group;
        const float scale = Elem<DT>::load(sz[(g * N + n) * 2]);
        const float zero = Elem<DT>::load(sz[(g * N + n) * 2 + 1]);
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) {
            const uint32_t w = wq[t4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int odd = 0; odd < 2; ++odd) {
                    const int64_t k = kt * 32 + 2 * t4 + 8 * j + odd;
                    if (k < K) {
                        const float code = static_cast<float>(static_cast<int>((w >> (4 * j + 16 * odd)) & 15u) - 8);
                        acc = __builtin_fmaf(Elem<DT>::load(xr[k]), __builtin_fmaf(code, scale, zero), acc);
                    }
                }
        }
    }
    red[t] = acc;
    __syncthreads();
    if (t < 8) {
        float s = 0.0f;
        for (int i = 0; i < 32; ++i) s += red[i * 8 + t];
        y[m * N + n] = Elem<DT>::store(s);
    }
}

template <int DT, int MROWS>
int launch_decode_rows(const void* x, const int32_t* packed, const void* sz, void* y, int N, int K,
                       int group, hipStream_t s) {
    const int k_super = K / 32;
    const dim3 grid((N + kWave - 1) / kWave), block(kDecodeWaves * kWave);
    const auto* xp = static_cast<const uint32_t*>(x);
    const auto* pp = reinterpret_cast<const uint4*>(packed);
    const auto* sp = static_cast<const uint32_t*>(sz);
    auto* yp = static_cast<uint16_t*>(y);
    switch (group) {
        case 32: int4_decode_kernel<DT, MROWS, 1><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super); break;
        case 64: int4_decode_kernel<DT, MROWS, 2><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super); break;
        default: int4_decode_kernel<DT, MROWS, 4><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super); break;
    }
    return check_launch("tpq_int4_mm (decode)");
}

template <int DT>
int launch_decode(const void* x, int64_t M, const int32_t* packed, const void* sz, void* y, int N,
                  int K, int group, hipStream_t s) {
    // rows go through in slabs of at most four; each slab streams the weight once
    const size_t row_bytes_x = static_cast<size_t>(K) * 2, row_bytes_y = static_cast<size_t>(N) * 2;
    for (int64_t m0 = 0; m0 < M; m0 += 4) {
        const int rows = static_cast<int>(M - m0 < 4 ? M - m0 : 4);
        const void* xs = static_cast<const char*>(x) + m0 * row_bytes_x;
        void* ys = static_cast<char*>(y) + m0 * row_bytes_y;
        int rc;
        switch (rows) {
            case 1: rc = launch_decode_rows<DT, 1>(xs, packed, sz, ys, N, K, group, s); break;
            case 2: rc = launch_decode_rows<DT, 2>(xs, packed, sz, ys, N, K, group, s); break;
            case 3: rc = launch_decode_rows<DT, 3>(xs, packed, sz, ys, N, K, group, s); break;
            default: rc = launch_decode_rows<DT, 4>(xs, packed, sz, ys, N, K, group, s); break;
        }
        if (rc != TPQ_OK) return rc;
    }
    return TPQ_OK;
}

template <int DT>
int launch_generic(const void* x, int64_t M, const int32_t* packed, const void* sz, void* y,
                   int64_t N, int64_t K, int64_t group, hipStream_t s) {
    using S = typename Elem<DT>::storage;
    const int64_t k_super = (K + 31) / 32;
    for (int64_t m0 = 0; m0 < M; m0 += 65535) {
        const int64_t rows = M - m0 < 65535 ? M - m0 : 65535;
        const dim3 grid(static_cast<unsigned>(N / 8), static_cast<unsigned>(rows));
        int4_generic_kernel<DT><<<grid, 256, 0, s>>>(static_cast<const S*>(x) + m0 * K,
                                                   reinterpret_cast<const uint32_t*>(packed),
                                                   static_cast<const S*>(sz),
                                                   static_cast<S*>(y) + m0 * N, N, K, k_super, group);
    }
    return check_launch("tpq_int4_mm (generic)");
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int tpq_int4_mm(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed,
                           int inner_k_tiles, int64_t N, int64_t group, const void* scales_and_zeros,
                           void* out, void* stream) {
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F32 || dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16,
                TPQ_ERR_INVALID_TYPE, "_weight_int4pack_mm(): activations must be floating point");
    TPQ_REQUIRE(group == 32 || group == 64 || group == 128, TPQ_ERR_INVALID_VALUE,
                "_weight_int4pack_mm(): qGroupSize must be 32, 64 or 128");
    TPQ_REQUIRE(inner_k_tiles == 2 || inner_k_tiles == 4 || inner_k_tiles == 8, TPQ_ERR_INVALID_VALUE,
                "_weight_int4pack_mm(): packed weight layout is invalid");
    // The reference's device kernel reads one word per lane, which is only the
    // layout written for innerKTiles = 2 (QuantGemmKernels.cu:1170-1202); its
    // Python callers always pack with 2 (int4_weight_only.py:94).
    TPQ_REQUIRE(inner_k_tiles == 2, TPQ_ERR_UNSUPPORTED,
                "_weight_int4pack_mm(): only innerKTiles = 2 packed weights are supported");
    TPQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && N % 8 == 0, TPQ_ERR_INVALID_VALUE,
                "_weight_int4pack_mm(): K dimension does not match packed B");
    if (M == 0 || N == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(x && packed && scales_and_zeros && out, TPQ_ERR_INVALID_VALUE,
                "_weight_int4pack_mm(): null pointer");
    TPQ_REQUIRE(N <= 0x7FFFFFF8 && K <= 0x7FFFFFE0, TPQ_ERR_INVALID_VALUE,
                "_weight_int4pack_mm(): dimension too large");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool fast = dtype != TPQ_DTYPE_F32 && K % 128 == 0 && aligned(x, 16) &&
                      aligned(packed, 16) && aligned(scales_and_zeros, 4) && aligned(out, 2);
    if (fast) {
        if (dtype == TPQ_DTYPE_F16)
            return launch_decode<TPQ_DTYPE_F16>(x, M, packed, scales_and_zeros, out, (int)N, (int)K, (int)group, s);
        return launch_decode<TPQ_DTYPE_BF16>(x, M, packed, scales_and_zeros, out, (int)N, (int)K, (int)group, s);
    }
    switch (dtype) {
        case TPQ_DTYPE_F32: return launch_generic<TPQ_DTYPE_F32>(x, M, packed, scales_and_zeros, out, N, K, group, s);
        case TPQ_DTYPE_F16: return launch_generic<TPQ_DTYPE_F16>(x, M, packed, scales_and_zeros, out, N, K, group, s);
        default: return launch_generic<TPQ_DTYPE_BF16>(x, M, packed, scales_and_zeros, out, N, K, group, s);
    }
}
