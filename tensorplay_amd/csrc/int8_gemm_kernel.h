// int8 x int8 -> int32 GEMM on the gfx950 matrix cores, with the dequant
// epilogue of the dynamic-activation int8 linear fused in.
//
//   acc[m,n] = sum_k a[m,k] * w[n,k]           (both operands K-contiguous)
//   out[m,n] = cast((float(acc) * rs[m]) * cs[n] (+ bias[n]))     or raw int32
//
// Tiling (one 256-thread workgroup = 4 wavefronts per output tile):
//   workgroup tile BM x BN = 256 x 128, k-step 64 bytes;
//   wavefront tile 128 x 64 = 4 x 2 blocks of v_mfma_i32_32x32x32_i8
//   (128 int32 accumulators per lane);
//   LDS holds two stages of (BM + BN) rows x 64 bytes.  A lane's MFMA operand
//   is 16 consecutive k of one row, i.e. one 16-byte chunk: chunks are stored
//   at position (chunk ^ swz(row)) inside their row so that both the 16-byte
//   stores (4 lanes per row) and the 16-byte fragment reads (one row per lane)
//   spread over all banks.
//   Global -> register -> LDS staging: while the matrix cores work on stage s
//   the next 64 k of both operands are already in flight into registers.
//
// With M = 2048, N = 4096 this is 8 x 32 = 256 tiles: one per compute unit.
#pragma once
#include <type_traits>

#include "tpq_common.h"

namespace tpq {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;             // bytes of k per stage
constexpr int kChunksPerRow = 4;    // 16-byte chunks per row per stage

__device__ __forceinline__ int swz(int row) { return (((row >> 1) ^ (row >> 3)) & 1) | (((row >> 2) & 1) << 1); }

struct EpilogueInt32 {
    int32_t* c;
    __device__ __forceinline__ void store(int64_t idx, int m, int n, int v) const { c[idx] = v; }
    // the two-step form of the scaled epilogues: nothing to fetch here
    __device__ __forceinline__ float row_scale_of(int) const { return 0.0f; }
    __device__ __forceinline__ float col_scale_of(int) const { return 0.0f; }
    __device__ __forceinline__ float bias_of(int) const { return 0.0f; }
    __device__ __forceinline__ void store_scaled(int64_t idx, int v, float, float, float) const { c[idx] = v; }
    // `count` (1..4) consecutive channels n .. of row m
    __device__ __forceinline__ void store_run(int64_t idx, int m, int n, const int (&v)[4], int count) const {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < count) c[idx + e] = v[e];
    }
};

template <int DT>
struct EpilogueDequant {
    typename Elem<DT>::storage* out;
    const float* rs;
    const float* cs;
    const float* bias;
    __device__ __forceinline__ void store(int64_t idx, int m, int n, int v) const {
        float f = __fmul_rn(__fmul_rn(static_cast<float>(v), rs[m]), cs[n]);
        if (bias) f = __fadd_rn(f, bias[n]);
        out[idx] = Elem<DT>::store(f);
    }
    // The same in two steps, for kernels that know early what they will store: the scales are fetched ahead of the
    // arithmetic instead of behind it, where the fetch is a trip to memory that nothing covers.
    __device__ __forceinline__ float row_scale_of(int m) const { return rs[m]; }
    __device__ __forceinline__ float col_scale_of(int n) const { return cs[n]; }
    __device__ __forceinline__ float bias_of(int n) const { return bias ? bias[n] : 0.0f; }
    __device__ __forceinline__ void store_scaled(int64_t idx, int v, float r, float c, float b) const {
        float f = __fmul_rn(__fmul_rn(static_cast<float>(v), r), c);
        if (bias) f = __fadd_rn(f, b);
        out[idx] = Elem<DT>::store(f);
    }
    // `count` (1..4) consecutive channels n .. of row m; every scale is fetched before the first store (a load behind a
    // store to `out` cannot be moved ahead of it, so store() in a loop waits for memory once per element)
    __device__ __forceinline__ void store_run(int64_t idx, int m, int n, const int (&v)[4], int count) const {
        const float r = rs[m];
        float c[4], b[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            c[e] = cs[e < count ? n + e : n];
            b[e] = bias ? bias[e < count ? n + e : n] : 0.0f;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float f = __fmul_rn(__fmul_rn(static_cast<float>(v[e]), r), c[e]);
            if (bias) f = __fadd_rn(f, b[e]);
            if (e < count) out[idx + e] = Elem<DT>::store(f);
        }
    }
};

// BitNet: out = cast((float(acc) * rs[m]) * w_scale (+ bias[n])), optionally the raw sums too.
template <int DT>
struct EpilogueTernary {
    typename Elem<DT>::storage* out;
    int32_t* acc_out;
    const float* rs;
    const float* bias;
    float w_scale;
    __device__ __forceinline__ void store(int64_t idx, int m, int n, int v) const {
        if (acc_out) acc_out[idx] = v;
        if (out) {
            float f = __fmul_rn(__fmul_rn(static_cast<float>(v), rs[m]), w_scale);
            if (bias) f = __fadd_rn(f, bias[n]);
            out[idx] = Elem<DT>::store(f);
        }
    }
    // The same in two steps, for kernels that store many elements per lane: the scale and the bias are fetched
    // first (a load after a store to `out` cannot be moved ahead of it by the compiler, so store() in a loop
    // waits for memory once per element).
    __device__ __forceinline__ float row_scale_of(int m) const { return out ? rs[m] : 0.0f; }
    __device__ __forceinline__ float bias_of(int n) const { return out && bias ? bias[n] : 0.0f; }
    __device__ __forceinline__ void store_scaled(int64_t idx, int v, float row_scale, float bias_n) const {
        if (acc_out) acc_out[idx] = v;
        if (out) {
            float f = __fmul_rn(__fmul_rn(static_cast<float>(v), row_scale), w_scale);
            if (bias) f = __fadd_rn(f, bias_n);
            out[idx] = Elem<DT>::store(f);
        }
    }
    // Four consecutive columns of one row (idx = m N + n).  whole_and_aligned: all four exist and idx is a multiple of
    // four with runs_aligned() true, so each destination takes one vector store.
    __device__ __forceinline__ bool runs_aligned() const {
        return (reinterpret_cast<uintptr_t>(out) & (4 * sizeof(typename Elem<DT>::storage) - 1)) == 0 && (reinterpret_cast<uintptr_t>(acc_out) & 15) == 0;
    }
    __device__ __forceinline__ void store_scaled_run(int64_t idx, const int (&v)[4], float row_scale, const float (&bias_n)[4], int count,
                                                     bool whole_and_aligned) const {
        if (acc_out) {
            if (whole_and_aligned) {
                *reinterpret_cast<int4*>(acc_out + idx) = make_int4(v[0], v[1], v[2], v[3]);
            } else {
                for (int e = 0; e < count; ++e) acc_out[idx + e] = v[e];
            }
        }
        if (out) {
            typename Elem<DT>::storage o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float f = __fmul_rn(__fmul_rn(static_cast<float>(v[e]), row_scale), w_scale);
                if (bias) f = __fadd_rn(f, bias_n[e]);
                o[e] = Elem<DT>::store(f);
            }
            if (whole_and_aligned) {
                if constexpr (sizeof(typename Elem<DT>::storage) == 2) {
                    *reinterpret_cast<uint2*>(out + idx) = make_uint2(o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16));
                } else {
                    *reinterpret_cast<float4*>(out + idx) = make_float4(o[0], o[1], o[2], o[3]);
                }
            } else {
                for (int e = 0; e < count; ++e) out[idx + e] = o[e];
            }
        }
    }
};

// One packed byte holds four ternary codes, first code in bits 7..6
// (tensorplay/ao/quantization/bitnet.py:75-79).  Expands it to four int8 in
// memory order, sign-extending each 2-bit field like the reference's unpack
// (0b11 -> -1, 0b10 -> -2).
__device__ __forceinline__ uint32_t ternary_byte_to_i8x4(uint32_t b) {
    uint32_t d = ((b >> 6) & 3u) | (((b >> 4) & 3u) << 8) | (((b >> 2) & 3u) << 16) | ((b & 3u) << 24);
    const uint32_t neg = (d >> 1) & 0x01010101u;
    return d | (neg * 0xFCu);
}

__device__ __forceinline__ uint4 ternary_word_to_i8x16(uint32_t w) {
    return make_uint4(ternary_byte_to_i8x4(w & 0xFFu), ternary_byte_to_i8x4((w >> 8) & 0xFFu),
                      ternary_byte_to_i8x4((w >> 16) & 0xFFu), ternary_byte_to_i8x4(w >> 24));
}

// TERNARY_W: W is the 2-bit packed matrix [N, K/4]; a 16-code chunk is one 32-bit word.
// DEPTH: k-stages held in registers ahead of the one being multiplied.  With small tiles a stage
// is little arithmetic, and one stage of lookahead leaves the global-load latency exposed in
// every iteration.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool TERNARY_W, class Epilogue, int DEPTH = 1>
__global__ __launch_bounds__(WAVES_M* WAVES_N* kWave) void int8_gemm_nk_kernel(
    const int8_t* __restrict__ A, const int8_t* __restrict__ W, int M, int N, int K, Epilogue ep) {
    constexpr int kThreads = WAVES_M * WAVES_N * kWave;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int kRows = BM + BN;
    constexpr int kLoadsA = BM * kChunksPerRow / kThreads;
    constexpr int kLoadsB = BN * kChunksPerRow / kThreads;
    static_assert(BM * kChunksPerRow % kThreads == 0 && BN * kChunksPerRow % kThreads == 0, "tile/threads");

    __shared__ uint4 lds[2][kRows * kChunksPerRow];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // tile order: consecutive workgroups walk down M inside one N panel, so the
    // workgroups resident together share few distinct W panels
    const int tiles_m = (M + BM - 1) / BM;
    const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int k_chunks = K >> 4;  // K % 16 == 0
    const int stages = (K + kBK - 1) / kBK;

    // global -> register staging: thread t moves chunk (t % 4) of row (t / 4 + i * kThreads/4)
    const int ld_chunk = tid & 3, ld_row = tid >> 2;
    using BChunk = typename std::conditional<TERNARY_W, uint32_t, uint4>::type;
    const uint4* a_src[kLoadsA];
    const BChunk* b_src[kLoadsB];
#pragma unroll
    for (int i = 0; i < kLoadsA; ++i) {
        int r = m0 + ld_row + i * (kThreads / 4);
        r = r < M ? r : M - 1;
        a_src[i] = reinterpret_cast<const uint4*>(A + static_cast<size_t>(r) * K) + ld_chunk;
    }
#pragma unroll
    for (int i = 0; i < kLoadsB; ++i) {
        int r = n0 + ld_row + i * (kThreads / 4);
        r = r < N ? r : N - 1;
        b_src[i] = reinterpret_cast<const BChunk*>(W + static_cast<size_t>(r) * (TERNARY_W ? K / 4 : K)) + ld_chunk;
    }
    uint4 ra_ring[DEPTH][kLoadsA];
    BChunk rb_ring[DEPTH][kLoadsB];
    auto fetch = [&](int stage, uint4 (&ra)[kLoadsA], BChunk (&rb)[kLoadsB]) {
        const int kc = stage * kChunksPerRow + ld_chunk;
        const bool in = kc < k_chunks;  // also false for stages past the end
#pragma unroll
        for (int i = 0; i < kLoadsA; ++i) ra[i] = in ? a_src[i][stage * kChunksPerRow] : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < kLoadsB; ++i) rb[i] = in ? b_src[i][stage * kChunksPerRow] : BChunk{};
    };
    auto stash = [&](int buf, const uint4 (&ra)[kLoadsA], const BChunk (&rb)[kLoadsB]) {
#pragma unroll
        for (int i = 0; i < kLoadsA; ++i) {
            const int r = ld_row + i * (kThreads / 4);
            lds[buf][r * kChunksPerRow + (ld_chunk ^ swz(r))] = ra[i];
        }
#pragma unroll
        for (int i = 0; i < kLoadsB; ++i) {
            const int r = BM + ld_row + i * (kThreads / 4);
            if constexpr (TERNARY_W)
                lds[buf][r * kChunksPerRow + (ld_chunk ^ swz(r))] = ternary_word_to_i8x16(rb[i]);
            else
                lds[buf][r * kChunksPerRow + (ld_chunk ^ swz(r))] = rb[i];
        }
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

#pragma unroll
    for (int d = 0; d < DEPTH; ++d) fetch(d, ra_ring[d], rb_ring[d]);
    stash(0, ra_ring[0], rb_ring[0]);
    fetch(DEPTH, ra_ring[0], rb_ring[0]);
    __syncthreads();

    // stage t waits in ring slot t % DEPTH
    const int frag_row = lane & 31, frag_half = lane >> 5;
    for (int s0 = 0; s0 < stages; s0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int s = s0 + d;
        if (s >= stages) break;
        const int buf = s & 1;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int chunk = ks * 2 + frag_half;
            v4i fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int r = wm * WM + i * 32 + frag_row;
                fa[i] = __builtin_bit_cast(v4i, lds[buf][r * kChunksPerRow + (chunk ^ swz(r))]);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int r = BM + wn * WN + j * 32 + frag_row;
                fb[j] = __builtin_bit_cast(v4i, lds[buf][r * kChunksPerRow + (chunk ^ swz(r))]);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (s + 1 < stages) {
            stash(buf ^ 1, ra_ring[(d + 1) % DEPTH], rb_ring[(d + 1) % DEPTH]);
            fetch(s + 1 + DEPTH, ra_ring[(d + 1) % DEPTH], rb_ring[(d + 1) % DEPTH]);
            __syncthreads();
        }
      }
    }

    // C fragment of a 32x32 block: lane holds column lane%32, rows 8*(v/4) + 4*(lane/32) + v%4
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * WN + j * 32 + frag_row;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm * WM + i * 32 + 8 * (v >> 2) + 4 * frag_half + (v & 3);
                if (m < M && n < N) ep.store(static_cast<int64_t>(m) * N + n, m, n, acc[i][j][v]);
            }
        }
}

inline bool mfma_path_ok(const void* a, const void* w, int64_t M, int64_t N, int64_t K) {
    return K % 16 == 0 && K >= 16 && aligned(a, 16) && aligned(w, 16) && M <= 0x7FFFFFFF &&
           N <= 0x7FFFFFFF && K <= 0x7FFFFFFF;
}

template <bool TERNARY_W = false, class Epilogue>
int launch_mfma(const int8_t* a, const void* w, int64_t M, int64_t N, int64_t K, Epilogue ep,
                hipStream_t s) {
    const auto* wp = static_cast<const int8_t*>(w);
    const int m = static_cast<int>(M), n = static_cast<int>(N), k = static_cast<int>(K);
    if (M > 128) {
        constexpr int BM = 256, BN = 128;
        const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
        TPQ_REQUIRE(tiles <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "int8 gemm: too many tiles");
        int8_gemm_nk_kernel<BM, BN, 2, 2, TERNARY_W, Epilogue>
            <<<dim3(static_cast<unsigned>(tiles)), 256, 0, s>>>(a, wp, m, n, k, ep);
    } else if (((M + 127) / 128) * ((N + 63) / 64) >= 512) {  // short activations: narrower tiles, more of them
        constexpr int BM = 128, BN = 64;
        const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
        TPQ_REQUIRE(tiles <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "int8 gemm: too many tiles");
        int8_gemm_nk_kernel<BM, BN, 4, 1, TERNARY_W, Epilogue, 2>
            <<<dim3(static_cast<unsigned>(tiles)), 256, 0, s>>>(a, wp, m, n, k, ep);
    } else {  // too few of those to fill the chip: 64 x 32 tiles, two wavefronts each
        constexpr int BM = 64, BN = 32;
        const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
        int8_gemm_nk_kernel<BM, BN, 2, 1, TERNARY_W, Epilogue, 4>
            <<<dim3(static_cast<unsigned>(tiles)), 128, 0, s>>>(a, wp, m, n, k, ep);
    }
    return check_launch("int8 mfma gemm");
}

}  // namespace
}  // namespace tpq
