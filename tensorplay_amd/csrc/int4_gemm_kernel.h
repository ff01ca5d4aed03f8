// int4 weight-only GEMM for many activation rows (prefill, large decode batches): fp16 / bf16, K % 128 == 0,
// N % 8 == 0, groups of 32, 64 or 128.  The packed weight is read once per 128 rows and never written
// back dense.
//
// A workgroup owns 128 activation rows (8 blocks of 16) x 16 NB WAVES channels and walks K in steps of
// 128.  Weights take the decode kernel's route: lane (i, q) of a wavefront owns channel row i of its NB blocks
// and k-tile 4 s + q, one 16-byte load per block and step straight into registers, unpacked in place and
// dequantized there with the roundings of the reference's dense weight, T(code - 8) * scale + zero
// (int4_tc_dequantize_kernel, p10/src/backend/cuda/QuantGemmKernels.cu:1170-1202): they are the A operand of
// v_mfma_f32_16x16x32.  The activations of a step (128 rows x 128 k, 32 KB) go through LDS, double buffered, one
// barrier per step: every wavefront needs all of them, as B operands, once per channel block.  A row is 256
// bytes + 16 of padding, so the sixteen lanes of a fragment read (row m, 16 bytes at 64 q + 16 u) hit
// sixteen different groups of four banks.  Lane (m, q) of the result holds row 16 rb + m, channels 4 q + v of a
// block; sums stay in the MFMA accumulators over the whole K range (fp32) and are rounded once at the end.
//
// Few rows (one or two tiles of 128) leave most compute units without a workgroup: N / 64 workgroups, 64 of them at
// N = 4096.  With a workspace the steps of K are dealt to gridDim.z slices; every slice leaves its fp32 sums in the
// workspace and int4_gemm_finish_kernel adds the slices in order and rounds once, so the result does not depend on how
// the launch was scheduled.
#pragma once

#include <atomic>
#include <type_traits>

#include "int4_mfma_kernel.h"

namespace tpq {
namespace {

constexpr int kGemmRows = 128;                 // activation rows per workgroup
constexpr int kGemmRowBlocks = kGemmRows / 16;
constexpr int kGemmPitch = 256 + 16;           // bytes per activation row of a step in LDS
constexpr int kGemmStageBytes = kGemmRows * kGemmPitch;

// One unpacked pair (two codes as 16-bit floats with the magic offset) -> the dense weight's two values, with the
// roundings of the reference's dequantize kernel: T(code - 8) * scale rounded to T, + zero rounded to T.
template <int DT>
struct DensePair;
template <>
struct DensePair<TPQ_DTYPE_F16> {
    half2_t s2, z2;
    __device__ __forceinline__ explicit DensePair(uint32_t pw)
        : s2(__builtin_bit_cast(half2_t, (pw & 0xFFFFu) | (pw << 16))), z2(__builtin_bit_cast(half2_t, (pw >> 16) | (pw & 0xFFFF0000u))) {}
    __device__ __forceinline__ uint32_t operator()(uint32_t pv, bool odd) const {
        const half2_t off_even = {static_cast<_Float16>(1032.0f), static_cast<_Float16>(1032.0f)};  // magic + 8
        const half2_t off_odd = {static_cast<_Float16>(72.0f), static_cast<_Float16>(72.0f)};
        const half2_t code = __builtin_bit_cast(half2_t, pv) - (odd ? off_odd : off_even);  // exact
        return __builtin_bit_cast(uint32_t, code * s2 + z2);  // packed fp16: rounded after the product and after the sum
    }
};
template <>
struct DensePair<TPQ_DTYPE_BF16> {
    // bf16 has no packed arithmetic: both roundings in fp32.  A pair is (128 + code) twice; (code - 8) * scale =
    // fma(128 + code, scale, -136 scale) exactly (products of 8-bit mantissas), rounded to bf16 by v_cvt_pk_bf16_f32; then
    // + zero in fp32 and the second rounding.
    float sc, zero, shift;
    __device__ __forceinline__ explicit DensePair(uint32_t pw)
        : sc(bf16_bits_to_f32(pw & 0xFFFFu)), zero(bf16_bits_to_f32(pw >> 16)), shift(-136.0f * bf16_bits_to_f32(pw & 0xFFFFu)) {}
    __device__ __forceinline__ uint32_t operator()(uint32_t pv, bool) const {
        typedef float f2_t __attribute__((ext_vector_type(2)));
        typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
        const f2_t prod = {__builtin_fmaf(__builtin_bit_cast(float, pv << 16), sc, shift),
                           __builtin_fmaf(__builtin_bit_cast(float, pv & 0xFFFF0000u), sc, shift)};
        const uint32_t pr = __builtin_bit_cast(uint32_t, __builtin_convertvector(prod, bf2_t));
        const f2_t sum = {__builtin_bit_cast(float, pr << 16) + zero, __builtin_bit_cast(float, pr & 0xFFFF0000u) + zero};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(sum, bf2_t));
    }
};

// RSPLIT: the wavefronts of a workgroup form RSPLIT groups that share the channels and split the eight row blocks
// (each dequantizes the weights again, but there are RSPLIT times the wavefronts per SIMD to overlap loads, vector
// work and MFMAs when the grid is small).
template <int DT, int NB, int WAVES, int GKT, int RSPLIT>
__global__ __launch_bounds__(WAVES * kWave) void int4_gemm_kernel(const uint16_t* __restrict__ x, const uint4* __restrict__ packed,
                                                                 const uint32_t* __restrict__ sz, uint16_t* __restrict__ y, int M, int N,
                                                                 int K, int steps_per_slice, float* __restrict__ partial) {
    using L = Lane16<DT>;
    using ML = MfmaLane<DT>;
    constexpr int kThreads = WAVES * kWave;
    constexpr int kChunks = kGemmRows * 16 / kThreads;  // 16-byte chunks of a stage per thread: 8 or 4
    extern __shared__ uint4 gemm_lds[];                  // [2][128 rows][272 bytes]
    char* lds = reinterpret_cast<char*>(gemm_lds);

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int k_super = K / 32, n_tiles = N / 8;
    const int s_begin = blockIdx.z * steps_per_slice;                                            // this slice: steps s_begin .. steps - 1
    const int steps = K / 128 < s_begin + steps_per_slice ? K / 128 : s_begin + steps_per_slice;  // (every slice has at least one)
    constexpr int kChannelWaves = WAVES / RSPLIT, kRowBlocks = kGemmRowBlocks / RSPLIT;
    const int cw = wave % kChannelWaves, rp = wave / kChannelWaves;    // channel position, row part
    const int n0 = blockIdx.x * (16 * NB * kChannelWaves) + cw * (16 * NB);  // first channel of this wavefront
    const int m0 = blockIdx.y * kGemmRows;
    const int rows_here = M - m0 < kGemmRows ? M - m0 : kGemmRows;

    const uint4* w_base[NB];
    const uint32_t* sz_base[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int n = n0 + 16 * b + i;
        int tile = n >> 3;
        tile = tile < n_tiles ? tile : n_tiles - 1;  // channels past N: any valid tile, result dropped
        w_base[b] = packed + (static_cast<size_t>(tile) * k_super + q) * 8 + (i & 7);
        sz_base[b] = sz + (n < N ? n : N - 1);       // (scale, zero) of this lane's channel
    }
    // activation chunks of this thread: chunk c = j * kThreads + tid of the stage -> row c / 16, 16-byte column c % 16
    const uint4* x_src[kChunks];
    int x_dst[kChunks];
    bool x_live[kChunks];
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
        const int c = j * kThreads + tid, row = c >> 4, col = c & 15;
        x_live[j] = row < rows_here;
        x_src[j] = reinterpret_cast<const uint4*>(x + static_cast<size_t>(m0 + (x_live[j] ? row : 0)) * K) + col;
        x_dst[j] = row * kGemmPitch + col * 16;
    }
    const int frag_base = (rp * kRowBlocks * 16 + i) * kGemmPitch + q * 64;  // + rb * 16 * pitch + u * 16

    uint32_t magic_even, magic_odd;  // kept in VGPRs behind an opaque move: v_and_or_b32 takes one literal only
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_even) : "s"(L::kMagicEven));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_odd) : "s"(L::kMagicOdd));

    struct Weights {
        uint4 w[NB];
        uint32_t p[NB];
    };
    auto load_w = [&](int s, Weights& st) __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            st.w[b] = nt_load(w_base[b] + static_cast<size_t>(s) * 32);
            st.p[b] = sz_base[b][static_cast<size_t>((4 * s + q) / GKT) * N];
        }
    };
    uint4 xr[2][kChunks];  // two steps of activations on their way to LDS
    auto load_x = [&](int s, int set) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) xr[set][j] = x_live[j] ? x_src[j][s * 16] : make_uint4(0, 0, 0, 0);
    };
    auto store_x = [&](int set, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) *reinterpret_cast<uint4*>(lds + buf * kGemmStageBytes + x_dst[j]) = xr[set][j];
    };

    float4_t acc[NB][kRowBlocks];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int rb = 0; rb < kRowBlocks; ++rb) acc[b][rb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // (always_inline: a call would put every captured array into scratch memory)
    auto compute = [&](const Weights& st, int buf) __attribute__((always_inline)) {
        uint32_t v[NB][4][4];  // [block][word r][pair j] = weights at k = 2 r + 8 j, + 1 of the lane's k-tile
#pragma unroll
        for (int b = 0; b < NB; ++b) {
#pragma unroll
            for (int r = 0; r < 4; ++r) L::template unpack<true>(dword_of(st.w[b], r), v[b][r], magic_even, magic_odd);
            const DensePair<DT> dense(st.p[b]);
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j) v[b][r][j] = dense(v[b][r][j], (j & 1) != 0);
        }
        const char* stage = lds + buf * kGemmStageBytes + frag_base;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int rb = 0; rb < kRowBlocks; ++rb) {  // rows past M are zeros in LDS: no branch, so the reads run ahead of the MFMAs
                const uint4 f = *reinterpret_cast<const uint4*>(stage + rb * (16 * kGemmPitch) + u * 16);
                const word4_t xb = {f.x, f.y, f.z, f.w};
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    const word4_t aw = {v[b][0][u], v[b][1][u], v[b][2][u], v[b][3][u]};
                    acc[b][rb] = ML::mfma(aw, xb, acc[b][rb]);
                }
            }
        }
    };

    // Four steps per trip with every index a constant: weights in a ring of four (loaded four steps ahead),
    // activations in two register sets (loaded two steps before they are stored to the stage that the step after
    // reads).  No branch around any load: steps past the end repeat the last one (loaded, stored to a stage nobody
    // reads, dropped), so every wait counts a fixed number of loads in flight.
    const int last = steps - 1;
    auto clamp = [&](int s) __attribute__((always_inline)) { return s < last ? s : last; };
    Weights wr[4] = {};
#pragma unroll
    for (int r = 0; r < 4; ++r) load_w(clamp(s_begin + r), wr[r]);
    load_x(s_begin, 0);
    store_x(0, 0);
    load_x(clamp(s_begin + 1), 1);
    load_x(clamp(s_begin + 2), 0);
    // LDS traffic only: __syncthreads() would also wait for the global loads in flight, which are the prefetch
    auto lds_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    lds_barrier();
    auto phase = [&](int s, auto pc) __attribute__((always_inline)) {
        constexpr int P = decltype(pc)::value;            // s % 4
        constexpr int buf = P & 1, set = (P + 1) & 1;     // stage of x(s); register set of x(s + 1)
        if (s < steps) compute(wr[P], buf);
        load_w(clamp(s + 4), wr[P]);
        store_x(set, buf ^ 1);  // stage buf ^ 1 was last read before the previous barrier
        load_x(clamp(s + 3), set);
        lds_barrier();
    };
    for (int s = s_begin; s < steps; s += 4) {
        phase(s, std::integral_constant<int, 0>{});
        phase(s + 1, std::integral_constant<int, 1>{});
        phase(s + 2, std::integral_constant<int, 2>{});
        phase(s + 3, std::integral_constant<int, 3>{});
    }

    // lane (m, q): row m0 + 16 rb + m, channels n0 + 16 b + 4 q + v
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int n = n0 + 16 * b + 4 * q;
        if (n >= N) continue;  // N % 8 == 0 and n % 4 == 0: all four channels exist
#pragma unroll
        for (int rb = 0; rb < kRowBlocks; ++rb) {
            const int row = 16 * (rp * kRowBlocks + rb) + i;
            if (row < rows_here) {
                const float4_t d = acc[b][rb];
                if (partial != nullptr) {  // this slice's sums: [slice][M][N] fp32
                    *reinterpret_cast<float4_t*>(partial + (static_cast<size_t>(blockIdx.z) * M + m0 + row) * N + n) = d;
                    continue;
                }
                const uint32_t lo = L::out(d[0]) | (static_cast<uint32_t>(L::out(d[1])) << 16);
                const uint32_t hi = L::out(d[2]) | (static_cast<uint32_t>(L::out(d[3])) << 16);
                *reinterpret_cast<uint2*>(y + static_cast<size_t>(m0 + row) * N + n) = make_uint2(lo, hi);
            }
        }
    }
}

// y = round(sum over the slices, in slice order); a thread takes four consecutive elements
template <int DT>
__global__ __launch_bounds__(256) void int4_gemm_finish_kernel(const float* __restrict__ partial, int slices, int64_t quads, uint16_t* __restrict__ y) {
    using L = Lane16<DT>;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= quads) return;
    // four slices requested together (a loop of load and add would wait for memory once per slice), added in slice
    // order; a batch past the last slice asks for the last one again and leaves it out of the sum
    float4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int z0 = 0; z0 < slices; z0 += 4) {
        float4_t more[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) more[j] = reinterpret_cast<const float4_t*>(partial)[static_cast<int64_t>(z0 + j < slices ? z0 + j : slices - 1) * quads + e];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (z0 + j < slices) sum = float4_t{sum[0] + more[j][0], sum[1] + more[j][1], sum[2] + more[j][2], sum[3] + more[j][3]};
    }
    const uint32_t lo = L::out(sum[0]) | (static_cast<uint32_t>(L::out(sum[1])) << 16);
    const uint32_t hi = L::out(sum[2]) | (static_cast<uint32_t>(L::out(sum[3])) << 16);
    reinterpret_cast<uint2*>(y)[e] = make_uint2(lo, hi);
}

// Slices of K for the tiled kernel (1: no workspace used).  `room`: bytes for the fp32 sums.  Chosen by an estimate
// of the time (us) fitted to measurements at 113 .. 255 rows (workgroups of 64 channels): a workgroup takes 5 + 7.2 per
// 1024 k of its slice; up to one workgroup per compute unit they all run at once, up to two per compute unit the pairs
// cost 1.7 times one, and so on; the second launch costs 1.6 + its bytes (slices x M x N x 4, written and read) at
// 4 TB/s.  Measured (one slice -> the choice): 4096 x 4096 at 128 rows 33.1 -> 19.7 (four slices), 11008 -> 4096
// 82.7 -> 34.3 (four), 8192 x 8192 62.7 -> 44.2 (two), 13824 -> 5120 at 192 rows 102 -> 74 (three); 4096 -> 11008 stays
// at one slice (35.3; two: 40.4).
struct Int4GemmPlan {
    int slices;
    double us;  // the estimate
};
inline Int4GemmPlan int4_gemm_plan(int64_t M, int64_t N, int64_t K, size_t room, int compute_units = 256) {
    const double tiles = static_cast<double>(((N + 63) / 64) * ((M + kGemmRows - 1) / kGemmRows));
    auto estimate = [&](int64_t slices) {
        const double per_unit = tiles * static_cast<double>(slices) / compute_units;
        const double rounds = per_unit <= 1.0 ? 1.0 : 1.7 * static_cast<double>(static_cast<int64_t>((per_unit + 1.999) / 2.0));
        const double main_us = rounds * (5.0 + 7.2 * static_cast<double>(K) / 1024.0 / static_cast<double>(slices));
        return main_us + (slices == 1 ? 0.0 : 1.6 + static_cast<double>(slices) * M * N * 8.0 / 4e6);
    };
    if (M > 256 || K < 1024) return {1, estimate(1)};
    const int64_t steps = K / 128, most = steps / 4 < 16 ? steps / 4 : 16;
    auto fits = [&](int64_t slices) { return slices == 1 || static_cast<size_t>(slices) * M * N * sizeof(float) <= room; };
    if (const char* e = tuning_env("TPQ_INT4_GEMM_SLICES")) {
        const int forced = std::atoi(e);
        return forced >= 1 && forced <= steps && fits(forced) ? Int4GemmPlan{forced, estimate(forced)} : Int4GemmPlan{1, estimate(1)};
    }
    Int4GemmPlan best{1, estimate(1)};
    for (int64_t slices = 2; slices <= most && fits(slices); ++slices)
        if (estimate(slices) < best.us) best = {static_cast<int>(slices), estimate(slices)};
    return best;
}
inline int int4_gemm_slices(int64_t M, int64_t N, int64_t K, size_t room) { return int4_gemm_plan(M, N, K, room).slices; }

// From how many rows the tiled kernel takes a shape: always from kInt4GemmRows; from kInt4GemmRowsSliced where its
// estimate is below that of the slabs of 32 rows it replaces, each of which streams the weight again: a slab of 32 rows
// takes about 2.7 + 0.37 per MB of packed weight + 0.67 per 1024 k (us, fitted to eight shapes, +- 10 %), a shorter last
// slab 45 % of that plus its share of the rest.  Measured (us, slabs / tiled, 33 - 48 - 64 - 80 - 96 - 112 rows):
//   4096 x 4096     12.1 13.9 15.8 21.2 23.0 28.3 / 15.0 15.5 16.0 16.8 17.6 18.3
//   4096 -> 11008   18.7 19.7 23.8 29.9 33.2 40.5 / 34.0 33.2 33.1 33.3 33.5 33.9
//   11008 -> 4096   24.4 28.8 33.1 43.5 47.5 58.8 / 29.5 29.2 29.6 30.0 31.0 31.5
//   8192 x 8192     27.9 29.7 34.3 45.0 49.6 60.9 / 38.8 38.5 38.1 38.7 39.6 40.1
//   2048 x 2048      8.8  9.8 10.8 14.8 15.6 19.9 /  9.8 10.0 10.4 10.8 11.2 11.7
//   13824 -> 5120   39.2 41.1 49.0 65.7 73.4 89.8 / 38.8 39.7 40.5 41.6 42.0 42.4
//   4096 -> 32000   43.0 49.8 57.4 73.2 81.5 98.4 / 54.9 52.4 51.9 51.9 50.2 52.5
//   5120 x 5120     17.2 19.0 22.8 30.2 34.1 41.3 / 20.6 20.7 21.3 22.1 22.6 23.6
constexpr int64_t kInt4GemmRows = 113, kInt4GemmRowsSliced = 33;
inline bool int4_gemm_takes(int64_t M, int64_t N, int64_t K, size_t room) {
    if (M >= kInt4GemmRows) return true;
    if (M < kInt4GemmRowsSliced) return false;
    const double slab = 2.7 + 0.37 * static_cast<double>(N) * static_cast<double>(K) / 2e6 + 0.67 * static_cast<double>(K) / 1024.0;
    const int64_t whole = M / 32, rest = M % 32;
    const double slabs = static_cast<double>(whole) * slab + (rest ? slab * (0.45 + 0.55 * static_cast<double>(rest) / 32.0) : 0.0);
    return int4_gemm_plan(M, N, K, room).us < slabs;
}

inline bool int4_gemm_ok(const void* x, const void* packed, const void* sz, const void* y, int64_t M, int64_t N, int64_t K, int64_t group) {
    return M >= 1 && N >= 8 && N % 8 == 0 && K >= 128 && K % 128 == 0 && (group == 32 || group == 64 || group == 128) && aligned(x, 16) &&
           aligned(packed, 16) && aligned(sz, 4) && aligned(y, 8) && M <= 0x7FFFFF00 && N <= 0x7FFFFF00 && K <= 0x7FFFFF00 &&
           (M + kGemmRows - 1) / kGemmRows <= 65535;
}

template <int DT, int NB, int WAVES, int RSPLIT>
int launch_int4_gemm_shape(const void* x, const int32_t* packed, const void* sz, void* y, int64_t M, int64_t N, int64_t K, int group,
                           int slices, float* partial, hipStream_t s) {
    constexpr size_t smem = 2 * static_cast<size_t>(kGemmStageBytes);
    constexpr int kChannels = 16 * NB * (WAVES / RSPLIT);
    const int steps_per_slice = static_cast<int>((K / 128 + slices - 1) / slices);
    slices = static_cast<int>((K / 128 + steps_per_slice - 1) / steps_per_slice);  // no empty slice
    if (slices == 1) partial = nullptr;
    const dim3 grid(static_cast<unsigned>((N + kChannels - 1) / kChannels), static_cast<unsigned>((M + kGemmRows - 1) / kGemmRows),
                    static_cast<unsigned>(slices));
    const auto* xp = static_cast<const uint16_t*>(x);
    const auto* pp = reinterpret_cast<const uint4*>(packed);
    const auto* sp = static_cast<const uint32_t*>(sz);
    auto* yp = static_cast<uint16_t*>(y);
#define TPQ_GEMM4(GKTV)                                                                                                      \
    {                                                                                                                        \
        auto kernel = int4_gemm_kernel<DT, NB, WAVES, GKTV, RSPLIT>;                                                                 \
        static std::atomic<uint64_t> configured{0};                                                                          \
        if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), smem, configured, "int4 gemm")) return rc;    \
        kernel<<<grid, WAVES * kWave, smem, s>>>(xp, pp, sp, yp, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), \
                                                 steps_per_slice, partial);                                                   \
    }
    if (group == 32) TPQ_GEMM4(1) else if (group == 64) TPQ_GEMM4(2) else TPQ_GEMM4(4)
#undef TPQ_GEMM4
    if (int rc = check_launch("tpq_int4_mm (gemm)")) return rc;
    if (partial == nullptr) return TPQ_OK;
    const int64_t quads = M * N / 4;  // N % 8 == 0
    int4_gemm_finish_kernel<DT><<<static_cast<unsigned>((quads + 255) / 256), 256, 0, s>>>(partial, slices, quads, yp);
    return check_launch("tpq_int4_mm (gemm, sum of the slices)");
}

template <int DT>
int launch_int4_gemm(const void* x, const int32_t* packed, const void* sz, void* y, int64_t M, int64_t N, int64_t K, int group, hipStream_t s,
                     int slices = 1, float* partial = nullptr) {
    static const int forced_nb = [] { const char* e = tuning_env("TPQ_INT4_GEMM_NB"); return e ? std::atoi(e) : 0; }();
    static const int forced_waves = [] { const char* e = tuning_env("TPQ_INT4_GEMM_WAVES"); return e ? std::atoi(e) : 0; }();
    static const int forced_rsplit = [] { const char* e = tuning_env("TPQ_INT4_GEMM_RSPLIT"); return e ? std::atoi(e) : 0; }();
    // Eight wavefronts per workgroup.  Few workgroups (up to 256 rows): two groups of four share the channels and split
    // the rows, 64 channels per workgroup while that gives at most one workgroup per compute unit, else 128; more rows:
    // 256 channels, which halves the LDS reads per product.  Measured (us, fp16): 4096 -> 11008: 128 rows 37.5 (42.2
    // without the split), 256 rows 53.9 with 128 channels (62.6 with 64), 512 rows 74.3 (98.1 with 64 channels);
    // 8192 x 8192, 256 rows: 73 with 64 channels (256 workgroups), 93 with 128.
    const bool few = M <= 256;
    const int64_t narrow_groups = ((N + 63) / 64) * ((M + kGemmRows - 1) / kGemmRows);
    const int nb = forced_nb ? forced_nb : (few && (narrow_groups <= 256 || slices > 1) ? 1 : 2);
    const int waves = forced_waves ? forced_waves : 8;
    const int rsplit = forced_rsplit ? forced_rsplit : (few ? 2 : 1);
    if (rsplit == 4 && waves == 16) {
        if (nb == 2) return launch_int4_gemm_shape<DT, 2, 16, 4>(x, packed, sz, y, M, N, K, group, slices, partial, s);
        return launch_int4_gemm_shape<DT, 1, 16, 4>(x, packed, sz, y, M, N, K, group, slices, partial, s);
    }
    if (rsplit == 2 && waves == 16) {
        if (nb == 2) return launch_int4_gemm_shape<DT, 2, 16, 2>(x, packed, sz, y, M, N, K, group, slices, partial, s);
        return launch_int4_gemm_shape<DT, 1, 16, 2>(x, packed, sz, y, M, N, K, group, slices, partial, s);
    }
    if (rsplit == 2) {
        if (nb == 2) return launch_int4_gemm_shape<DT, 2, 8, 2>(x, packed, sz, y, M, N, K, group, slices, partial, s);
        return launch_int4_gemm_shape<DT, 1, 8, 2>(x, packed, sz, y, M, N, K, group, slices, partial, s);
    }
    if (nb == 2 && waves == 8) return launch_int4_gemm_shape<DT, 2, 8, 1>(x, packed, sz, y, M, N, K, group, slices, partial, s);
    if (nb == 2) return launch_int4_gemm_shape<DT, 2, 4, 1>(x, packed, sz, y, M, N, K, group, slices, partial, s);
    return launch_int4_gemm_shape<DT, 1, 4, 1>(x, packed, sz, y, M, N, K, group, slices, partial, s);
}

}  // namespace
}  // namespace tpq
