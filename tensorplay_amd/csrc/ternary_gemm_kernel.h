// Ternary-weight GEMM for a block of up to 128 activation rows (BitNet prefill
// chunks, M = 9..128 per launch), K % 256 == 0.
//
// The work is small (M = 128, N = 2560, K = 6912 is 4.5 GOP, about a
// microsecond of matrix-core time) and there are few output tiles, so what
// matters is the length of the serial chain per tile: global load -> expand the
// 2-bit codes -> LDS -> barrier -> fragment reads -> MFMA.  A workgroup of 16
// wavefronts owns a BM x 32 output tile (BM = 128 or 64) and takes 256 bytes of k
// per stage: wavefront (mb, kp) multiplies rows 32 mb .. +31 with part kp of the
// stage (a quarter = two MFMAs for BM = 128, an eighth = one MFMA for BM = 64),
// so a tile needs K / 256 barriers instead of K / 64, and the k-parts are added
// through LDS at the end.  BM = 64 doubles the number of workgroups: it is used
// when 128-row tiles would leave most compute units idle (N = 2560: 80 tiles).
//
// LDS stage: BM activation rows + 32 weight rows, 256 bytes each, the sixteen
// 16-byte chunks of a row stored at position chunk ^ (row % 16) (conflict-free
// fragment reads).  Activations move as 16-byte chunks, two (one for BM = 64) per
// thread and stage; the packed weights as 32-bit words (16 codes = one int8
// chunk), one per thread for the first 512 threads.  Both are held in registers
// one stage ahead.
#pragma once

#include <cstdlib>

#include "int8_gemm_kernel.h"

namespace tpq {
namespace {

constexpr int kTgN = 32, kTgStage = 256, kTgThreads = 1024;
constexpr int kTgRowChunks = kTgStage / 16;  // 16

template <int BM, class Epilogue>
__global__ __launch_bounds__(kTgThreads) void ternary_gemm_m128_kernel(const int8_t* __restrict__ x,
                                                                       const uint8_t* __restrict__ packed,
                                                                       int M, int N, int K, Epilogue ep) {
    constexpr int kTgM = BM;
    constexpr int kTgBufChunks = (kTgM + kTgN) * kTgRowChunks;  // 2560 chunks = 40 KB (BM = 128), 24 KB (BM = 64)
    constexpr int kMBlocks = BM / 32, kParts = 16 / kMBlocks;   // wavefronts = m-blocks x k-parts
    constexpr int kPartChunks = kTgRowChunks / kParts;          // 16-byte chunks of a k-part: 4 or 2
    extern __shared__ uint4 tg_lds[];  // [2][kTgBufChunks], later the k-part partial sums
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int mb = wave % kMBlocks, kq = wave / kMBlocks;
    const int n0 = blockIdx.x * kTgN, m0 = blockIdx.y * kTgM;
    const int stages = K / kTgStage;

    // activations: chunks tid and (BM = 128) tid + 1024 of the stage -> row c / 16, 16-byte chunk c % 16
    // (plain scalars, not arrays: the staging registers must not end up in scratch memory)
    const int ch = tid & 15, row0 = tid >> 4, row1 = BM == 128 ? row0 + 64 : row0;
    const int gr0 = m0 + row0 < M ? m0 + row0 : M - 1, gr1 = m0 + row1 < M ? m0 + row1 : M - 1;
    const uint4* a_src0 = reinterpret_cast<const uint4*>(x + static_cast<size_t>(gr0) * K) + ch;
    const uint4* a_src1 = reinterpret_cast<const uint4*>(x + static_cast<size_t>(gr1) * K) + ch;
    const int a_dst0 = row0 * kTgRowChunks + (ch ^ (row0 & 15)), a_dst1 = row1 * kTgRowChunks + (ch ^ (row1 & 15));
    // weights: threads 0..511, row tid / 16, word tid % 16 (16 codes -> int8 chunk tid % 16)
    const bool w_loader = tid < kTgN * kTgRowChunks;
    const int grw = n0 + row0 < N ? n0 + row0 : N - 1;
    const uint32_t* w_src = reinterpret_cast<const uint32_t*>(packed + static_cast<size_t>(w_loader ? grw : 0) * (K / 4)) + ch;
    const int w_dst = (kTgM + (w_loader ? row0 : 0)) * kTgRowChunks + (ch ^ (row0 & 15));
    uint4 ra0, ra1 = make_uint4(0, 0, 0, 0);
    uint32_t rw = 0;
#define TPQ_TG_FETCH(S)                              \
    do {                                             \
        ra0 = a_src0[(S) * kTgRowChunks];            \
        if (BM == 128) ra1 = a_src1[(S) * kTgRowChunks]; \
        if (w_loader) rw = w_src[(S) * kTgRowChunks]; \
    } while (0)
#define TPQ_TG_STASH(BUF)                                          \
    do {                                                           \
        uint4* dst = tg_lds + (BUF) * kTgBufChunks;                \
        dst[a_dst0] = ra0;                                         \
        if (BM == 128) dst[a_dst1] = ra1;                          \
        if (w_loader) dst[w_dst] = ternary_word_to_i8x16(rw);      \
    } while (0)

    v16i acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0;

    const int frag_row = lane & 31, frag_half = lane >> 5;
    const int a_row = mb * 32 + frag_row, w_row = kTgM + frag_row;
    TPQ_TG_FETCH(0);
    TPQ_TG_STASH(0);
    if (stages > 1) TPQ_TG_FETCH(1);
    __syncthreads();
    for (int s = 0; s < stages; ++s) {
        const uint4* buf = tg_lds + (s & 1) * kTgBufChunks;
#pragma unroll
        for (int ks = 0; ks < kPartChunks / 2; ++ks) {
            const int chunk = kq * kPartChunks + ks * 2 + frag_half;
            const v4i fa = __builtin_bit_cast(v4i, buf[a_row * kTgRowChunks + (chunk ^ (a_row & 15))]);
            const v4i fb = __builtin_bit_cast(v4i, buf[w_row * kTgRowChunks + (chunk ^ (w_row & 15))]);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc, 0, 0, 0);
        }
        if (s + 1 < stages) {
            TPQ_TG_STASH((s + 1) & 1);  // the other buffer: everybody finished reading it before the previous barrier
            if (s + 2 < stages) TPQ_TG_FETCH(s + 2);
            __syncthreads();
        }
    }

#undef TPQ_TG_FETCH
#undef TPQ_TG_STASH
    // add the k-parts: parts 1.. park their sums in LDS (15 x 4 KB at most), part 0 finishes the tile
    __syncthreads();
    int* part = reinterpret_cast<int*>(tg_lds);
    if (kq > 0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) part[(((kq - 1) * kMBlocks + mb) * 16 + v) * kWave + lane] = acc[v];
    }
    __syncthreads();
    if (kq == 0) {
#pragma unroll 1
        for (int q = 0; q < kParts - 1; ++q)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] += part[((q * kMBlocks + mb) * 16 + v) * kWave + lane];
        // C fragment of a 32x32 block: lane holds column lane%32, rows 8*(v/4) + 4*(lane/32) + v%4
        const int n = n0 + frag_row;
        if (n < N) {
            float row_scale[16];  // fetched before the first store: a load behind a store to `out` has to wait for it
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + mb * 32 + 8 * (v >> 2) + 4 * frag_half + (v & 3);
                row_scale[v] = ep.row_scale_of(m < M ? m : M - 1);
            }
            const float bias_n = ep.bias_of(n);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + mb * 32 + 8 * (v >> 2) + 4 * frag_half + (v & 3);
                if (m < M) ep.store_scaled(static_cast<int64_t>(m) * N + n, acc[v], row_scale[v], bias_n);
            }
        }
    }
}

inline bool ternary_gemm_m128_ok(int64_t M, int64_t K) { return M > 8 && K % kTgStage == 0; }

template <int BM, class Epilogue>
int launch_ternary_gemm_tile(const int8_t* x, const uint8_t* packed, int64_t M, int64_t N, int64_t K,
                             Epilogue ep, hipStream_t s) {
    // two stage buffers (80 KB / 48 KB); the k-part sums parked at the end reuse them and need
    // (16 - BM / 32) wavefronts x 4 KB (48 KB / 56 KB)
    constexpr size_t stage_bytes = 2 * static_cast<size_t>((BM + kTgN) * kTgRowChunks) * 16;
    constexpr size_t part_bytes = static_cast<size_t>(16 - BM / 32) * 16 * kWave * sizeof(int);
    constexpr size_t smem = stage_bytes > part_bytes ? stage_bytes : part_bytes;
    auto kernel = ternary_gemm_m128_kernel<BM, Epilogue>;
    static std::atomic<uint64_t> configured{0};  // per instantiation
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), smem, configured, "ternary gemm")) return rc;
    const int64_t gx = (N + kTgN - 1) / kTgN, gy = (M + BM - 1) / BM;
    TPQ_REQUIRE(gx <= 0x7FFFFFFF && gy <= 65535, TPQ_ERR_INVALID_VALUE, "ternary gemm: shape too large");
    kernel<<<dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)), kTgThreads, smem, s>>>(
        x, packed, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), ep);
    return check_launch("tpq_ternary_mm (gemm)");
}

template <class Epilogue>
int launch_ternary_gemm_m128(const int8_t* x, const uint8_t* packed, int64_t M, int64_t N, int64_t K,
                             Epilogue ep, hipStream_t s) {
    // 64-row tiles for up to 64 rows (128-row tiles would be half empty: 8192 -> 28672 at 64 rows 63 us against 85,
    // 4096 x 4096 12.3 against 14.2) and when 128-row tiles would occupy at most half of the 256 compute units
    // (4096 x 4096 at 128 rows: 13.8 us against 15.7; 2560 -> 6912, 216 tiles: 14.7 against 13.1, stays on 128)
    const int64_t tiles128 = ((N + kTgN - 1) / kTgN) * ((M + 127) / 128);
    static const int forced = [] { const char* e = tuning_env("TPQ_TERNARY_BM"); return e ? atoi(e) : 0; }();
    const bool small = forced ? forced == 64 : (M <= 64 || tiles128 <= 128);
    return small ? launch_ternary_gemm_tile<64>(x, packed, M, N, K, ep, s) : launch_ternary_gemm_tile<128>(x, packed, M, N, K, ep, s);
}

}  // namespace
}  // namespace tpq
