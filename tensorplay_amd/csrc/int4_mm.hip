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
//     (w & 0x000F000F) | 0x64006400 is the fp16 pair (1024+c, 1024+c), (w & 0x00F000F0) | 0x54005400 is (64+c, 64+c)
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
#include <cstdlib>

#include "int4_flight.h"
#include "int4_lane.h"
#include "int4_mfma_kernel.h"
#include "int4_gemm_kernel.h"
#include "int4_row_kernel.h"

namespace tpq {
namespace {

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
//
// WPB wavefronts per workgroup; gridDim.y = KS workgroups share one column group, each taking
// every (WPB*KS)-th chunk.  With KS > 1 the workgroups leave their partial columns in
// ws_part[KS][MROWS][N] and bump ws_count[column group]; the one that arrives last adds the KS
// partials in slice order (so the result does not depend on arrival order), stores y and puts
// the counter back to zero.  Partials and counter move with agent-scope atomic accesses, which
// are coherent across the chip's L2 slices.
// CPW > 0: every wavefront owns exactly CPW chunks (K = 128 x WPB x CPW, one workgroup per column group) and the code
// from the first load to the LDS exchange is free of branches: all loads are issued up front, the small ones first,
// and the k-tiles are consumed one by one as they arrive.  With a loop and its bounds checks around the chunks
// (CPW = 0) the compiler waits for every outstanding load before the first use, which leaves the whole
// arithmetic of the wavefront (two chunks: about 400 vector instructions) behind the end of the stream.
// PAUSE > 0: the wavefront sleeps 64 x PAUSE clocks between the requests of its first chunk and those of the others.
// The memory system takes a compute unit's requests at the rate it returns data, oldest wavefront first, so without the
// pause wavefront 0 has asked for everything before wavefront 15 has asked for anything, the chunks of the last
// wavefronts all arrive at the very end, and their arithmetic (a quarter of a SIMD's work) trails the stream.  With
// it every wavefront's first chunk is asked for ahead of the second chunks and only half of that work is left at
// the end.  Measured at 4096 -> 11008 (us): no pause 6.19; 12: 6.12; 16..24: 6.05..6.07; 32: 6.29; 40: 6.43.
template <int DT, int MROWS, int GROUP_KT, int WPB, int CPW = 0, int PAUSE = 0>
__global__ __launch_bounds__(WPB* kWave) void int4_decode_kernel(
    const uint32_t* __restrict__ x, const uint4* __restrict__ packed, const uint32_t* __restrict__ sz,
    uint16_t* __restrict__ y, int N, int K, int k_super, float* ws_part, unsigned* ws_count) {
    using L = Lane16<DT>;
    constexpr int kGroups = kChunkKT / GROUP_KT;
    __shared__ float red[WPB * MROWS * kWave];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = WPB == 1 ? 0 : __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = blockIdx.x * kWave + lane;
    const int n_ld = n < N ? n : N - 1;  // lanes past the edge read a valid column and drop the result
    const uint4* wp = packed + (static_cast<size_t>(n_ld >> 3) * k_super) * 8 + (n_ld & 7);
    const uint32_t* szp = sz + n_ld;
    const int words_per_row = K >> 1;
    const int n_chunks = k_super / kChunkKT;

    uint32_t magic_even, magic_odd;  // kept in VGPRs: v_and_or_b32 takes one scalar operand only
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_even) : "s"(L::kMagicEven));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_odd) : "s"(L::kMagicOdd));

    auto issue = [&](Chunk<MROWS, kGroups>& ch, int chunk) {
        chunk = chunk < n_chunks ? chunk : n_chunks - 1;  // past the end: harmless re-read, never used
#pragma unroll
        for (int i = 0; i < kChunkKT; ++i) ch.q[i] = nt_load(wp + static_cast<size_t>(chunk * kChunkKT + i) * 8);
#pragma unroll
        for (int g = 0; g < kGroups; ++g) ch.p[g] = nt_load(szp + static_cast<size_t>(chunk * kGroups + g) * N);
#pragma unroll
        for (int m = 0; m < MROWS; ++m) ch.xw[m] = x[static_cast<size_t>(m) * words_per_row + chunk * 64 + lane];
    };

    float yacc[MROWS];
#pragma unroll
    for (int m = 0; m < MROWS; ++m) yacc[m] = 0.0f;

    auto consume = [&](const Chunk<MROWS, kGroups>& ch, int chunk) {
        // Sums of the activations per k-tile and pair parity.  Lane l holds word l%16 of k-tile
        // l/16, i.e. pair j = (l%16)/4: adding across lane bits 0, 1 and 3 leaves the sum over
        // even pairs in lanes with bit 2 clear and the sum over odd pairs in those with it set.
        float xs[MROWS];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
            float s = L::dot(ch.xw[m], L::kOnes, 0.0f);
            s += __shfl_xor(s, 1, kWave);
            s += __shfl_xor(s, 2, kWave);
            s += __shfl_xor(s, 8, kWave);
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
            for (int t4 = 0; t4 < 4; ++t4) L::template unpack<false>(wq[t4], v[t4], magic_even, magic_odd);
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
                    float sx_even = 0.0f, sx_odd = 0.0f;
#pragma unroll
                    for (int g = 0; g < GROUP_KT; ++g) {
                        const int l0 = 16 * (i + 1 - GROUP_KT + g);
                        sx_even += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xs[m]), l0));
                        sx_odd += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xs[m]), l0 + 4));
                    }
                    float dotp = __builtin_fmaf(-L::kOffsetEven, sx_even, part[m]);
                    dotp = __builtin_fmaf(-L::kOffsetOdd, sx_odd, dotp);
                    yacc[m] = __builtin_fmaf(scale, dotp, yacc[m]);
                    yacc[m] = __builtin_fmaf(zero, sx_even + sx_odd, yacc[m]);
                    part[m] = 0.0f;
                }
            }
            // keep the k-tiles in program order: without this the scheduler unpacks
            // every tile of the chunk up front and runs out of registers
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int slices = CPW > 0 ? 1 : gridDim.y;
    if constexpr (CPW > 0) {
        Chunk<MROWS, kGroups> own[CPW];
        // (scale, zero) words and this lane's activation word of every chunk first: loads return in issue order, and
        // the sums of the activations are the first thing a chunk needs
#pragma unroll
        for (int u = 0; u < CPW; ++u) {
            const int chunk = wave + u * WPB;
#pragma unroll
            for (int m = 0; m < MROWS; ++m) own[u].xw[m] = x[static_cast<size_t>(m) * words_per_row + chunk * 64 + lane];
#pragma unroll
            for (int g = 0; g < kGroups; ++g) own[u].p[g] = nt_load(szp + static_cast<size_t>(chunk * kGroups + g) * N);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < CPW; ++u) {
#pragma unroll
            for (int i = 0; i < kChunkKT; ++i) own[u].q[i] = nt_load(wp + static_cast<size_t>((wave + u * WPB) * kChunkKT + i) * 8);
            if constexpr (PAUSE > 0) {
                if (u == 0 && CPW > 1) {
                    __builtin_amdgcn_sched_barrier(0);
                    __builtin_amdgcn_s_sleep(PAUSE);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < CPW; ++u) consume(own[u], wave + u * WPB);
    } else {
    const int stride = WPB * slices;                 // chunks between two turns of this wavefront
    const int first = blockIdx.y * WPB + wave;
    Chunk<MROWS, kGroups> ring[kRing];
#pragma unroll
    for (int u = 0; u < kRing; ++u) issue(ring[u], first + u * stride);
    // Steady state without a branch in the body: a condition around a request makes every later wait a wait for all
    // outstanding loads, the chunk just asked for included.  Then the chunks that are left, at most 2 kRing - 1.
    int c = first;
    for (; c + (2 * kRing - 1) * stride < n_chunks; c += kRing * stride) {
#pragma unroll
        for (int u = 0; u < kRing; ++u) {
            consume(ring[u], c + u * stride);
            issue(ring[u], c + (kRing + u) * stride);
        }
    }
#pragma unroll
    for (int r = 0; r < 2 * kRing - 1; ++r) {
        const int cu = c + r * stride;
        if (cu < n_chunks) {
            consume(ring[r % kRing], cu);
            if (cu + kRing * stride < n_chunks) issue(ring[r % kRing], cu + kRing * stride);
        }
    }
    }

    // wavefronts of the workgroup meet in LDS
    if (WPB > 1) {
#pragma unroll
        for (int m = 0; m < MROWS; ++m) red[(wave * MROWS + m) * kWave + lane] = yacc[m];
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int m = 0; m < MROWS; ++m) {
                float s = 0.0f;
#pragma unroll
                for (int w = 0; w < WPB; ++w) s += red[(w * MROWS + m) * kWave + lane];
                yacc[m] = s;
            }
        }
    }
    if (slices == 1) {
        if (wave == 0 && n < N) {
#pragma unroll
            for (int m = 0; m < MROWS; ++m) y[static_cast<size_t>(m) * N + n] = L::out(yacc[m]);
        }
        return;
    }
    // several workgroups per column group: leave the partial, count arrivals
    if (wave == 0) {
        if (n < N) {
#pragma unroll
            for (int m = 0; m < MROWS; ++m)
                __hip_atomic_store(ws_part + (static_cast<size_t>(blockIdx.y) * MROWS + m) * N + n, yacc[m],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // every lane's partial has reached the coherent level before lane 0 announces the arrival
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        unsigned seen = 0;
        if (lane == 0)
            seen = __hip_atomic_fetch_add(ws_count + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        seen = __builtin_amdgcn_readfirstlane(seen);
        if (seen == static_cast<unsigned>(slices - 1)) {  // last to arrive: fold in slice order
            if (n < N) {
#pragma unroll
                for (int m = 0; m < MROWS; ++m) {
                    float s = 0.0f;
                    for (int ks = 0; ks < slices; ++ks)
                        s += __hip_atomic_load(ws_part + (static_cast<size_t>(ks) * MROWS + m) * N + n,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    y[static_cast<size_t>(m) * N + n] = L::out(s);
                }
            }
            if (lane == 0) __hip_atomic_store(ws_count + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace
}  // namespace tpq

#include "int4_stream_kernel.h"

namespace tpq {
namespace {

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

// Workspace handed in by the caller: kCounterSlots arrival counters (zero between calls),
// then the partial columns [KS][MROWS][N].
constexpr int kCounterSlots = 4096;
constexpr size_t kCounterBytes = kCounterSlots * sizeof(unsigned);

inline int compute_units() {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 256;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
        return n;
    }();
    return cus;
}

struct DecodePlan {
    int wpb;     // wavefronts per workgroup
    int slices;  // workgroups per column group (1 = no workspace needed)
};

// Each wavefront should own about two chunks (256 k of 64 columns); beyond one workgroup of 16
// wavefronts per column group the k range is sliced across workgroups, which lets all compute
// units share the columns evenly when there are few column groups.
inline DecodePlan plan_decode(int N, int K, int mrows, size_t workspace_bytes) {
    const int n_chunks = K / 128;
    const int col_groups = (N + kWave - 1) / kWave;
    DecodePlan plan{kDecodeWaves, 1};
    const char* env_wpb = tuning_env("TPQ_INT4_WPB");
    const char* env_ks = tuning_env("TPQ_INT4_KS");
    int wpb = 0, ks = 0;
    if (workspace_bytes > kCounterBytes && col_groups <= kCounterSlots) {
        const size_t per_slice = static_cast<size_t>(mrows) * N * sizeof(float);
        const int max_slices = static_cast<int>((workspace_bytes - kCounterBytes) / per_slice);
        // Slicing costs a trip through memory per workgroup (partials out, counter, partials in:
        // about 1.5 us measured), so it only pays when one workgroup per column group would
        // leave most of the chip idle.  TPQ_INT4_WPB / TPQ_INT4_KS override for experiments.
        if (env_wpb || env_ks) {
            wpb = env_wpb ? std::atoi(env_wpb) : 4;
            ks = env_ks ? std::atoi(env_ks) : (n_chunks + 2 * wpb - 1) / (2 * wpb);
        } else if (col_groups * 4 <= compute_units() && n_chunks >= 16) {
            wpb = 8;
            ks = 2;
        }
        if (ks > max_slices) ks = max_slices;
        if (ks > 64) ks = 64;
    }
    if (ks >= 2 && (wpb == 1 || wpb == 2 || wpb == 4 || wpb == 8 || wpb == 16)) plan = DecodePlan{wpb, ks};
    if (const char* e = tuning_env("TPQ_INT4_WPB1")) plan = DecodePlan{std::atoi(e), 1};  // wavefronts per workgroup without slices (sweeps)
    return plan;
}

template <int DT, int MROWS, int WPB>
int launch_decode_rows(const void* x, const int32_t* packed, const void* sz, void* y, int N, int K,
                       int group, int slices, void* workspace, hipStream_t s) {
    const int k_super = K / 32;
    const dim3 grid((N + kWave - 1) / kWave, slices), block(WPB * kWave);
    const auto* xp = static_cast<const uint32_t*>(x);
    const auto* pp = reinterpret_cast<const uint4*>(packed);
    const auto* sp = static_cast<const uint32_t*>(sz);
    auto* yp = static_cast<uint16_t*>(y);
    auto* counters = static_cast<unsigned*>(workspace);
    auto* partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + kCounterBytes);
    auto run = [&](auto gkt) {
        constexpr int G = decltype(gkt)::value;
        if (WPB == 16 && slices == 1 && !tuning_env("TPQ_DECODE_LOOP")) {  // the branch-free body where the chunks divide evenly
            const int n_chunks = K / 128;
            if (n_chunks == 16) { int4_decode_kernel<DT, MROWS, G, WPB, 1><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super, partials, counters); return; }
            if (n_chunks == 32) {
                if constexpr (MROWS == 1) {
                    static const bool no_pause = tuning_env("TPQ_INT4_NO_PAUSE") != nullptr;
                    if (!no_pause) { int4_decode_kernel<DT, MROWS, G, WPB, 2, 20><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super, partials, counters); return; }
                }
                int4_decode_kernel<DT, MROWS, G, WPB, 2><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super, partials, counters);
                return;
            }
            if (n_chunks == 48 && MROWS == 1 && G == 4) {
                static const bool no_pause3 = tuning_env("TPQ_INT4_NO_PAUSE") != nullptr;
                if (!no_pause3) { int4_decode_kernel<DT, MROWS, G, WPB, 3, 20><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super, partials, counters); return; }
                int4_decode_kernel<DT, MROWS, G, WPB, 3><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super, partials, counters);
                return;
            }
        }
        int4_decode_kernel<DT, MROWS, G, WPB><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, k_super, partials, counters);
    };
    switch (group) {
        case 32: run(std::integral_constant<int, 1>{}); break;
        case 64: run(std::integral_constant<int, 2>{}); break;
        default: run(std::integral_constant<int, 4>{}); break;
    }
    return check_launch("tpq_int4_mm (decode)");
}

template <int DT, int MROWS>
int launch_decode_plan(const void* x, const int32_t* packed, const void* sz, void* y, int N, int K,
                       int group, void* workspace, size_t workspace_bytes, hipStream_t s) {
    const DecodePlan plan = plan_decode(N, K, MROWS, workspace ? workspace_bytes : 0);
    switch (plan.wpb) {
        case 1: return launch_decode_rows<DT, MROWS, 1>(x, packed, sz, y, N, K, group, plan.slices, workspace, s);
        case 2: return launch_decode_rows<DT, MROWS, 2>(x, packed, sz, y, N, K, group, plan.slices, workspace, s);
        case 4: return launch_decode_rows<DT, MROWS, 4>(x, packed, sz, y, N, K, group, plan.slices, workspace, s);
        case 8: return launch_decode_rows<DT, MROWS, 8>(x, packed, sz, y, N, K, group, plan.slices, workspace, s);
        default: return launch_decode_rows<DT, MROWS, 16>(x, packed, sz, y, N, K, group, plan.slices, workspace, s);
    }
}

// One activation row through the streaming kernel; false if the shape does not fit it.
template <int DT>
bool launch_stream(const void* x, const int32_t* packed, const void* sz, void* y, int N, int K, int group,
                   hipStream_t s, int* rc) {
    // Measured on MI355X at M=1, K=4096, N=11008 the column-per-lane kernel is the faster of the
    // two (7.1 us against 8.3 us); the streaming kernel is kept selectable for comparison runs.
    const char* force = tuning_env("TPQ_INT4_KERNEL");
    if (!(force && force[0] == 's')) return false;  // TPQ_INT4_KERNEL=stream opts in
    const int k_super = K / 32, n_tiles = N / 8;
    int tiles_per_block = (n_tiles + compute_units() - 1) / compute_units();
    if (tiles_per_block > 8) tiles_per_block = 8;   // 16 wavefronts per workgroup at most
    const int waves = 2 * tiles_per_block;
    const size_t smem = sizeof(uint32_t) * (static_cast<size_t>(k_super) * (kXStride + 2) + waves * 8);
    if (smem > 64 * 1024) return false;
    const dim3 grid((n_tiles + tiles_per_block - 1) / tiles_per_block), block(waves * kWave);
    const auto* xp = static_cast<const uint32_t*>(x);
    const auto* pp = reinterpret_cast<const uint4*>(packed);
    const auto* sp = static_cast<const uint32_t*>(sz);
    auto* yp = static_cast<uint16_t*>(y);
#define TPQ_STREAM(GKT, EX) \
    int4_stream_kernel<DT, GKT, EX><<<grid, block, smem, s>>>(xp, pp, sp, yp, N, k_super, n_tiles, tiles_per_block)
    const bool exact = k_super % 16 == 0;
    switch (group) {
        case 32: if (exact) TPQ_STREAM(1, true); else TPQ_STREAM(1, false); break;
        case 64: if (exact) TPQ_STREAM(2, true); else TPQ_STREAM(2, false); break;
        default: if (exact) TPQ_STREAM(4, true); else TPQ_STREAM(4, false); break;
    }
#undef TPQ_STREAM
    *rc = check_launch("tpq_int4_mm (stream)");
    return true;
}

// Up to 16 rows per launch on the matrix cores; false if the shape does not fit that kernel.
// residual (may be null): [rows][N] added to the rounded output; it forces this kernel for one row too.
template <int DT>
bool launch_mfma_rows(const void* x, int rows, const int32_t* packed, const void* sz, void* y, int N, int K,
                      int group, hipStream_t s, int* rc, const void* residual = nullptr) {
    const bool deq = (group == 32 || group == 64) && residual == nullptr;  // dequantized in registers
    if ((group != 128 && group != 256 && !deq) || !aligned(sz, 16) || !aligned(y, 8)) return false;
    if (residual != nullptr && !aligned(residual, 8)) return false;
    const char* force = tuning_env("TPQ_INT4_KERNEL");  // "mfma" / "decode" pin the choice for comparison runs
    if (force && force[0] == 'd' && residual == nullptr) return false;
    // One row: the column-per-lane kernel wins only where N is wide enough to fill the chip with its
    // 64-column workgroups (measured: N = 11008, K = 4096: 7.1 us against 8.5 us here; N = 4096,
    // K = 11008: 12.5 against 9.7; N = 8192, K = 28672: 32.8 against 26.4).
    if (rows == 1 && residual == nullptr && N >= 10240 && !(force && force[0] == 'm')) return false;
    // Channels per workgroup (16 nb) and wavefronts per workgroup, from a sweep over model shapes
    // (K 4096..28672, 2..16 rows).  Every workgroup reads all of x from cache, so many rows want wide
    // workgroups, but only when N still yields enough of them to fill the chip:
    //   N <= 4096:  16 ch x 8 waves always (8 rows: 5.3 us against 6.0 for 32 ch, 8.5 for 64 ch)
    //   N = 4097 .. 10239:  32 ch x 8 waves (8192 x 8192, 8 rows: 9.8 us against 13.4 for 16 ch, 14.6 for 64 ch; N = 5120,
    //                320 workgroups of 16 ch on 256 compute units: 13824 -> 5120 at 8 rows 14.2 us against 21.1, 5120 x 5120 7.4 against 9.9)
    //   N = 10240 .. 28672:  64 ch x 8 waves up to 12 rows (4096 -> 11008: 8.0 / 8.1 / 8.4 / 9.0 us at 2 / 4 / 8 / 12
    //                rows against 8.4 / 8.5 / 9.0 / 9.3 for the next best; 8192 -> 28672, 8 rows: 27.4 against 30.4),
    //                64 ch x 4 waves above (16 rows: 9.7 us against 12.3 for 32 ch)
    //   N > 28672:   32 ch x 4 waves up to 4 rows, 64 ch x 4 waves above (4096 -> 32000, 4 rows: 16.2 against 16.6)
    if (!(force && force[0] == 'm')) {  // the all-in-flight form, where it is built and wins
        FlightWeights one{};
        one.packed[0] = packed; one.sz[0] = sz; one.y[0] = y; one.N[0] = N; one.count = 1;
        if (flight_launch(DT, x, rows, one, K, group, false, residual, s, rc)) return true;
    }
    const bool wide = N >= 10240 && N <= 28672 && rows <= 12;
    int nb = N > 4096 ? (N < 10240 ? 2 : (rows > 4 || wide ? 4 : 2)) : 1;
    if (const char* env = tuning_env("TPQ_INT4_NB")) nb = std::atoi(env);
    int waves = N < 10240 || wide ? 8 : 4;
    if (const char* env = tuning_env("TPQ_INT4_WAVES")) waves = std::atoi(env);
    const auto* xp = static_cast<const uint16_t*>(x);
    const auto* pp = reinterpret_cast<const uint4*>(packed);
    const auto* sp = static_cast<const uint32_t*>(sz);
    auto* yp = static_cast<uint16_t*>(y);
    const int shift = group == 128 ? 0 : 1;  // a group is 128 << shift k (128 or 256)
    {
        if (deq) {
#define TPQ_MFMA_DEQ(NBV, WV, GKTV)                                                                                       \
    int4_mfma_kernel<DT, NBV, WV, false, GKTV><<<dim3((N + 16 * NBV - 1) / (16 * NBV)), dim3(WV * kWave), 0, s>>>( \
        xp, pp, sp, yp, rows, N, K, 0, nullptr, nullptr, nullptr)
            // same shapes of workgroup as for groups of 128
            if (group == 32) {
                if (nb == 1) TPQ_MFMA_DEQ(1, 8, 1); else if (nb == 2 && waves == 8) TPQ_MFMA_DEQ(2, 8, 1);
                else if (nb == 2) TPQ_MFMA_DEQ(2, 4, 1); else TPQ_MFMA_DEQ(4, 4, 1);
            } else {
                if (nb == 1) TPQ_MFMA_DEQ(1, 8, 2); else if (nb == 2 && waves == 8) TPQ_MFMA_DEQ(2, 8, 2);
                else if (nb == 2) TPQ_MFMA_DEQ(2, 4, 2); else TPQ_MFMA_DEQ(4, 4, 2);
            }
#undef TPQ_MFMA_DEQ
            *rc = check_launch("tpq_int4_mm (mfma, small groups)");
            return true;
        }
    }
    if (rows > 16) {  // 17..32 rows: two row blocks per workgroup share the unpacked weights
        if (deq) return false;
#define TPQ_MFMA2(NBV, WV) \
    int4_mfma_kernel<DT, NBV, WV, false, 4, 2><<<dim3((N + 16 * NBV - 1) / (16 * NBV)), dim3(WV * kWave), 0, s>>>( \
        xp, pp, sp, yp, rows, N, K, shift, nullptr, nullptr, static_cast<const uint16_t*>(residual))
        if (nb == 1) TPQ_MFMA2(1, 8); else if (nb == 2 && waves == 8) TPQ_MFMA2(2, 8); else if (nb == 2) TPQ_MFMA2(2, 4); else TPQ_MFMA2(4, 4);
#undef TPQ_MFMA2
        *rc = check_launch("tpq_int4_mm (mfma, 32 rows)");
        return true;
    }
#define TPQ_MFMA(NBV, WV) \
    int4_mfma_kernel<DT, NBV, WV><<<dim3((N + 16 * NBV - 1) / (16 * NBV)), dim3(WV * kWave), 0, s>>>( \
        xp, pp, sp, yp, rows, N, K, shift, nullptr, nullptr, static_cast<const uint16_t*>(residual))
    if (waves == 16 && nb == 1) {
        TPQ_MFMA(1, 16);
    } else if (waves == 8) {
        if (nb == 1) TPQ_MFMA(1, 8); else if (nb == 2) TPQ_MFMA(2, 8); else TPQ_MFMA(4, 8);
    } else {
        if (nb == 1) TPQ_MFMA(1, 4); else if (nb == 2) TPQ_MFMA(2, 4); else TPQ_MFMA(4, 4);
    }
#undef TPQ_MFMA
    *rc = check_launch("tpq_int4_mm (mfma)");
    return true;
}

// gate / up pair with the SwiGLU epilogue, and the plain product plus a residual: slabs of 16 rows
template <int DT>
int launch_fused(const void* x, int64_t M, const int32_t* packed, const void* sz, const int32_t* packed_b, const void* sz_b,
                 const void* residual, void* y, int N, int K, int group, hipStream_t s, const void* norm_weight = nullptr,
                 float norm_eps = 0.0f) {
    const size_t row_x = static_cast<size_t>(K) * 2, row_y = static_cast<size_t>(N) * 2;
    for (int64_t m0 = 0; m0 < M; m0 += 16) {
        const int rows = static_cast<int>(M - m0 < 16 ? M - m0 : 16);
        const char* xs = static_cast<const char*>(x) + m0 * row_x;
        char* ys = static_cast<char*>(y) + m0 * row_y;
        int rc = TPQ_OK;
        if (packed_b != nullptr) {
            FlightWeights two{};
            two.packed[0] = packed; two.packed[1] = packed_b; two.sz[0] = sz; two.sz[1] = sz_b; two.y[0] = ys; two.N[0] = two.N[1] = N;
            two.count = 2;
            two.norm_weight = norm_weight;
            two.norm_eps = norm_eps;
            if (flight_launch(DT, xs, rows, two, K, group, true, nullptr, s, &rc)) {
                if (rc != TPQ_OK) return rc;
                continue;
            }
            if (norm_weight != nullptr) return fail(TPQ_ERR_UNSUPPORTED, "tpq_int4_mm_swiglu_norm: this shape is not built");
            static const int pair_waves = [] { const char* e = tuning_env("TPQ_INT4_PAIR_WAVES"); return e ? std::atoi(e) : 4; }();
            const auto* xp = reinterpret_cast<const uint16_t*>(xs);
            const auto* pa = reinterpret_cast<const uint4*>(packed);
            const auto* pb = reinterpret_cast<const uint4*>(packed_b);
            const auto* sa = static_cast<const uint32_t*>(sz);
            const auto* sb = static_cast<const uint32_t*>(sz_b);
            auto* yp = reinterpret_cast<uint16_t*>(ys);
            const dim3 grid((N + 15) / 16);
            if (pair_waves == 8)
                int4_mfma_kernel<DT, 2, 8, true><<<grid, dim3(8 * kWave), 0, s>>>(xp, pa, sa, yp, rows, N, K, group == 128 ? 0 : 1, pb, sb, nullptr);
            else
                int4_mfma_kernel<DT, 2, 4, true><<<grid, dim3(4 * kWave), 0, s>>>(xp, pa, sa, yp, rows, N, K, group == 128 ? 0 : 1, pb, sb, nullptr);
            rc = check_launch("tpq_int4_mm_swiglu");
        } else if (!launch_mfma_rows<DT>(xs, rows, packed, sz, ys, N, K, group, s, &rc, static_cast<const char*>(residual) + m0 * row_y)) {
            return fail(TPQ_ERR_UNSUPPORTED, "tpq_int4_mm_add: this shape or alignment is not built");
        }
        if (rc != TPQ_OK) return rc;
    }
    return TPQ_OK;
}

// Several weights, one launch per slab of 16 rows (see int4_mfma_multi_kernel).  The workgroup shape follows the
// rule of launch_mfma_rows for the sum of the widths: that is the width the chip sees.
template <int DT>
int launch_multi(const void* x, int64_t M, int count, const int32_t* const* packed, const int64_t* N, const void* const* sz,
                 void* const* y, int K, int group, hipStream_t s, const void* norm_weight = nullptr, float norm_eps = 0.0f) {
    int64_t n_total = 0;
    for (int w = 0; w < count; ++w) n_total += N[w];
    int64_t step = 16;
    for (int64_t m0 = 0; m0 < M; m0 += step) {
        step = 16;
        const int rows = static_cast<int>(M - m0 < 16 ? M - m0 : 16);
        {
            FlightWeights all{};
            all.count = count;
            for (int w = 0; w < count; ++w) {
                all.packed[w] = packed[w]; all.sz[w] = sz[w]; all.N[w] = static_cast<int>(N[w]);
                all.y[w] = static_cast<uint16_t*>(y[w]) + m0 * N[w];
            }
            all.norm_weight = norm_weight;
            all.norm_eps = norm_eps;
            int rc = TPQ_OK;
            // 17..32 rows left: one launch with two blocks of 16 rows, where the all-in-flight kernel is built for it
            const int rows32 = static_cast<int>(M - m0 < 32 ? M - m0 : 32);
            if (rows32 > 16 && norm_weight == nullptr &&
                flight_launch(DT, static_cast<const uint16_t*>(x) + m0 * K, rows32, all, K, group, false, nullptr, s, &rc)) {
                if (rc != TPQ_OK) return rc;
                step = 32;
                continue;
            }
            if (flight_launch(DT, static_cast<const uint16_t*>(x) + m0 * K, rows, all, K, group, false, nullptr, s, &rc)) {
                if (rc != TPQ_OK) return rc;
                continue;
            }
            if (norm_weight != nullptr) return fail(TPQ_ERR_UNSUPPORTED, "tpq_int4_mm_multi_norm: this shape is not built");
        }
        const bool wide = n_total >= 10240 && n_total <= 28672 && rows <= 12;
        const int nb = n_total > 4096 ? (n_total < 10240 ? 2 : (rows > 4 || wide ? 4 : 2)) : 1;
        const int waves = n_total < 10240 || wide ? 8 : 4;
        Int4MultiSet set{};
        set.count = count;
        int blocks = 0;
        for (int w = 0; w < count; ++w) {
            set.packed[w] = reinterpret_cast<const uint4*>(packed[w]);
            set.sz[w] = static_cast<const uint32_t*>(sz[w]);
            set.y[w] = static_cast<uint16_t*>(y[w]) + m0 * N[w];
            set.N[w] = static_cast<int>(N[w]);
            set.first[w] = blocks;
            blocks += static_cast<int>((N[w] + 16 * nb - 1) / (16 * nb));
        }
        set.first[count] = blocks;
        const auto* xp = static_cast<const uint16_t*>(x) + m0 * K;
        const int shift = group == 128 ? 0 : 1;
#define TPQ_MULTI(NBV, WV) int4_mfma_multi_kernel<DT, NBV, WV><<<dim3(blocks), dim3(WV * kWave), 0, s>>>(xp, set, rows, K, shift)
        if (waves == 8) { if (nb == 1) TPQ_MULTI(1, 8); else if (nb == 2) TPQ_MULTI(2, 8); else TPQ_MULTI(4, 8); }
        else { if (nb == 2) TPQ_MULTI(2, 4); else TPQ_MULTI(4, 4); }
#undef TPQ_MULTI
        if (int rc = check_launch("tpq_int4_mm_multi")) return rc;
    }
    return TPQ_OK;
}

// One activation row on the kernel that deals whole tiles of eight channels round-robin to one workgroup per compute
// unit (int4_row_kernel.h); false if the shape does not fit it.
template <int DT>
bool launch_row(const void* x, const int32_t* packed, const void* sz, void* y, int N, int K, int group, hipStream_t s, int* rc) {
    const char* force = tuning_env("TPQ_INT4_KERNEL");  // "row" pins it, any other value excludes it (sweeps)
    const int pinned = route_override_int4_row();
    if ((force && force[0] != 'r') || pinned == 0) return false;
    if (K % 256 != 0 || K > 16384 || N % 8 != 0) return false;  // four 1 KB blocks per wavefront and tile at most (registers)
    int cus = compute_units() / 32 * 32;
    if (cus < 32) cus = 32;
    const int n_tiles = N / 8;
    const int blocks = K / 256;
    const int seg = (blocks + kRowWaves - 1) / kRowWaves;
    const int waves = (blocks + seg - 1) / seg;  // <= 16; the last one may own a segment past K (zero activations)
    const int rounds = seg == 1 ? 6 : seg == 2 ? 3 : seg == 3 ? 2 : 1;
    // Where it wins (measured, one row, fp16, us: this kernel / matrix-core kernel / column-per-lane kernel):
    // 11008 -> 4096: 7.0 / 8.7 / 12.1;  5120 x 5120: 5.9 / 6.8 / 7.1.  Not for K <= 4096 (4096 -> 11008: 7.2 / 8.1 / 6.8;
    // 4096 x 4096: 6.0 / 4.7 / 5.8), not when the tiles need a second batch of rounds (4096 -> 14336: 10.1 / 8.6 / 7.7;
    // 8192 x 8192: 10.6 / 9.3 / 10.9), and a workgroup wants at least two tiles.
    // Wide weights (several batches of rounds per workgroup): this kernel deals tiles evenly to one workgroup per compute
    // unit, the column-per-lane kernel runs ceil(N / 64 / 256) rounds of workgroups and loses most where the last round
    // is a small fraction.  Measured (us, this kernel / default): K = 8192: N = 10240 10.5 / 11.6, 16384 14.9 / 16.7,
    // 20480 19.2 / 23.3, 28672 23.8 / 27.3 (14336: 14.5 / 14.7); K = 12288: N = 8192 11.6 / 12.8, 12288 15.9 / 17.1,
    // 24576 28.4 / 33.1; last round at most 60 % full (N = 20480, 24576): K = 5120 14.2 / 15.3, 7168 17.7 / 19.8,
    // 10240 22.1 / 25.7.  Elsewhere the default is as fast or faster (K = 5120, N = 14336: 11.1 / 9.1; K = 10240,
    // N = 14336: 17.9 / 15.5).
    const int column_groups = (N + kWave - 1) / kWave, last_round = column_groups % compute_units();
    const bool short_last_round = column_groups > compute_units() && last_round > 0 && last_round * 10 <= compute_units() * 6;
    const bool wide = K > 4096 && (short_last_round || (K >= 7680 && K < 10240 && N >= 10240) || (K >= 12288 && N >= 8192));
    // 12288 < K <= 16384 (four blocks per wavefront, one round in flight): ahead of the looped column-per-lane kernel or
    // level with it (us, this kernel / default): 13824 -> 5120 12.1 / 14.5, 16384 -> 4096 9.9 / 14.4, 14336 -> 4096 9.3 / 9.5,
    // 16384 -> 8192 17.0 / 16.7.
    const bool wins = K > 4096 && ((n_tiles >= 2 * cus && n_tiles <= rounds * cus) || wide || seg == 4);
    if (!(force || pinned == 1) && !wins) return false;
    const int shift = group == 32 ? 0 : group == 64 ? 1 : group == 128 ? 2 : 3;
    const dim3 grid(cus), block(waves * kWave);
    const auto* xp = static_cast<const uint16_t*>(x);
    const auto* pp = reinterpret_cast<const uint4*>(packed);
    const auto* sp = static_cast<const uint32_t*>(sz);
    auto* yp = static_cast<uint16_t*>(y);
    switch (seg) {
        case 1: int4_row_kernel<DT, 1, 1, 6><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, n_tiles, shift); break;
        case 2: int4_row_kernel<DT, 1, 2, 3><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, n_tiles, shift); break;
        case 3: int4_row_kernel<DT, 1, 3, 2><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, n_tiles, shift); break;
        default: int4_row_kernel<DT, 1, 4, 1><<<grid, block, 0, s>>>(xp, pp, sp, yp, N, K, n_tiles, shift); break;  // (two rounds do not fit the registers)
    }
    *rc = check_launch("tpq_int4_mm (row)");
    return true;
}

template <int DT>
int launch_decode(const void* x, int64_t M, const int32_t* packed, const void* sz, void* y, int N,
                  int K, int group, void* workspace, size_t workspace_bytes, hipStream_t s) {
    if (M == 1) {
        int rc;
        if (launch_row<DT>(x, packed, sz, y, N, K, group, s, &rc)) return rc;
        const char* force = tuning_env("TPQ_INT4_KERNEL");
        if (!force) {  // narrow weights: the all-in-flight matrix-core kernel
            FlightWeights one{};
            one.packed[0] = packed; one.sz[0] = sz; one.y[0] = y; one.N[0] = N; one.count = 1;
            if (flight_launch(DT, x, 1, one, K, group, false, nullptr, s, &rc)) return rc;
        }
    }
    // Many rows: the tiled kernel, the packed weight read once per 128 rows, from 113 rows on and from 33 where its
    // estimate beats the 32-row slabs below (int4_gemm_takes; TPQ_INT4_GEMM_ROWS pins the row count in sweeps).
    static const int64_t gemm_rows = [] { const char* e = tuning_env("TPQ_INT4_GEMM_ROWS"); return e ? std::atoll(e) : int64_t{0}; }();
    // few tiles: slices of K over the chip, their fp32 sums in the workspace behind the counters
    const size_t room = workspace != nullptr && workspace_bytes > kCounterBytes ? workspace_bytes - kCounterBytes : 0;
    if ((gemm_rows ? M >= gemm_rows : int4_gemm_takes(M, N, K, room)) && int4_gemm_ok(x, packed, sz, y, M, N, K, group)) {
        const int slices = int4_gemm_slices(M, N, K, room);
        float* partial = slices > 1 ? reinterpret_cast<float*>(static_cast<char*>(workspace) + kCounterBytes) : nullptr;
        return launch_int4_gemm<DT>(x, packed, sz, y, M, N, K, group, s, slices, partial);
    }
    {   // slabs of 32 rows (16 with groups of 32 / 64) on the matrix cores where the shape allows
        static const int slab_rows = [] { const char* e = tuning_env("TPQ_INT4_SLAB_ROWS"); return e ? std::atoi(e) : 32; }();
        const size_t row_x = static_cast<size_t>(K) * 2, row_y = static_cast<size_t>(N) * 2;
        const int slab = (group == 32 || group == 64) ? 16 : slab_rows;
        int64_t m0 = 0;
        while (m0 < M) {
            const int rows = static_cast<int>(M - m0 < slab ? M - m0 : slab);
            int rc;
            if (!launch_mfma_rows<DT>(static_cast<const char*>(x) + m0 * row_x, rows, packed, sz,
                                      static_cast<char*>(y) + m0 * row_y, N, K, group, s, &rc)) break;
            if (rc != TPQ_OK) return rc;
            m0 += rows;
        }
        if (m0 >= M) return TPQ_OK;
        x = static_cast<const char*>(x) + m0 * row_x;  // what is left (a single last row, or everything) takes the paths below
        y = static_cast<char*>(y) + m0 * row_y;
        M -= m0;
    }
    // rows go through in slabs of at most four; each slab streams the weight once
    const size_t row_bytes_x = static_cast<size_t>(K) * 2, row_bytes_y = static_cast<size_t>(N) * 2;
    for (int64_t m0 = 0; m0 < M; m0 += 4) {
        const int rows = static_cast<int>(M - m0 < 4 ? M - m0 : 4);
        const void* xs = static_cast<const char*>(x) + m0 * row_bytes_x;
        void* ys = static_cast<char*>(y) + m0 * row_bytes_y;
        int rc;
        if (rows == 1 && launch_stream<DT>(xs, packed, sz, ys, N, K, group, s, &rc)) {
            if (rc != TPQ_OK) return rc;
            continue;
        }
        switch (rows) {
            case 1: rc = launch_decode_plan<DT, 1>(xs, packed, sz, ys, N, K, group, workspace, workspace_bytes, s); break;
            case 2: rc = launch_decode_plan<DT, 2>(xs, packed, sz, ys, N, K, group, workspace, workspace_bytes, s); break;
            case 3: rc = launch_decode_plan<DT, 3>(xs, packed, sz, ys, N, K, group, workspace, workspace_bytes, s); break;
            default: rc = launch_decode_plan<DT, 4>(xs, packed, sz, ys, N, K, group, workspace, workspace_bytes, s); break;
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

// Dense [N, K] weight from the packed layout, W = T(code - 8) * scale + zero with the product and the
// sum each rounded to T (reference: int4_tc_dequantize_kernel, QuantGemmKernels.cu:1170-1202).
// Thread = (row, k-tile): one 16-byte load, 32 consecutive outputs.
template <int DT>
__global__ __launch_bounds__(256) void int4_dequantize_kernel(const uint4* __restrict__ packed,
                                                              const typename Elem<DT>::storage* __restrict__ sz,
                                                              typename Elem<DT>::storage* __restrict__ W, int64_t N,
                                                              int64_t K, int64_t k_super, int64_t group, int64_t total, int vector_stores) {
    using S = typename Elem<DT>::storage;
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total; idx += gridDim.x * 256ll) {
        const int r = static_cast<int>(idx & 7);
        const int64_t tile = idx >> 3, kT = tile % k_super, nT = tile / k_super;
        const int64_t n = nT * 8 + r;
        const uint4 q = packed[idx];
        const int64_t g = (kT * 32) / group;
        const float scale = Elem<DT>::load(sz[(g * N + n) * 2]), zero = Elem<DT>::load(sz[(g * N + n) * 2 + 1]);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        __attribute__((aligned(16))) S out[32];
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int odd = 0; odd < 2; ++odd) {
                    const int code = static_cast<int>((w[t4] >> (4 * j + 16 * odd)) & 15u);
                    const float prod = Elem<DT>::load(Elem<DT>::store(__fmul_rn(static_cast<float>(code - 8), scale)));
                    out[2 * t4 + 8 * j + odd] = Elem<DT>::store(__fadd_rn(prod, zero));
                }
        S* dst = W + n * K + kT * 32;
        if (vector_stores && kT * 32 + 32 <= K) {  // 64 or 128 contiguous, 16-byte aligned bytes
            uint4* dst16 = reinterpret_cast<uint4*>(dst);
            const uint4* src16 = reinterpret_cast<const uint4*>(out);
#pragma unroll
            for (int e = 0; e < static_cast<int>(32 * sizeof(S) / 16); ++e) dst16[e] = src16[e];
        } else if (kT * 32 + 32 <= K) {
#pragma unroll
            for (int e = 0; e < 32; ++e) dst[e] = out[e];
        } else {
            for (int e = 0; e < 32 && kT * 32 + e < K; ++e) dst[e] = out[e];
        }
    }
}

// The same dense weight with row-contiguous stores, for K % 32 == 0 and a 16-byte aligned destination.  A thread
// produces the E = 16 / sizeof(T) consecutive outputs of one 16-byte store: piece p of the 32 k of (row, k-tile).
// The P = 32 / E threads of a k-tile load the same 16 bytes (one request to the cache) and each cuts out its own
// nibbles; 32 consecutive threads cover 32 E consecutive k of one row, so every store instruction writes whole
// cache lines, and the eight rows of a tile are taken by the same workgroup, which reads each packed line once.
template <int DT>
__global__ __launch_bounds__(256) void int4_dequantize_rows_kernel(const uint4* __restrict__ packed,
                                                                   const typename Elem<DT>::storage* __restrict__ sz,
                                                                   typename Elem<DT>::storage* __restrict__ W, int N, int K,
                                                                   int k_super, int group_tiles, int chunks_per_row) {
    using S = typename Elem<DT>::storage;
    constexpr int E = 16 / sizeof(S), P = 32 / E, kTilesPerGroup = 32 / P;  // k-tiles per workgroup and row
    const int nT = blockIdx.x / chunks_per_row, chunk = blockIdx.x - nT * chunks_per_row;
    const int r = threadIdx.x >> 5, q = threadIdx.x & 31;
    const int kT = chunk * kTilesPerGroup + q / P, p = q % P;
    if (kT >= k_super) return;
    const int n = nT * 8 + r;
    const uint4 w = packed[(static_cast<size_t>(nT) * k_super + kT) * 8 + r];  // the line serves all eight rows: plain load
    const size_t szi = (static_cast<size_t>(kT / group_tiles) * N + n) * 2;
    const float scale = Elem<DT>::load(sz[szi]), zero = Elem<DT>::load(sz[szi + 1]);
    auto code_of = [&](int e) {
        // k = p E + e inside the tile sits in word (k % 8) / 2, nibble k / 8 (+ 4 for odd k)
        const int k = p * E + e;
        const int t4 = (k & 7) >> 1;
        const uint32_t word = t4 == 0 ? w.x : t4 == 1 ? w.y : t4 == 2 ? w.z : w.w;
        return static_cast<float>(static_cast<int>((word >> (4 * (k >> 3) + 16 * (k & 1))) & 15u) - 8);
    };
    uint32_t words[4];
    if constexpr (DT == TPQ_DTYPE_BF16) {
        // both roundings with the hardware's packed conversion (round to nearest even); a NaN takes the
        // pattern 0x7FC0 that the scalar conversion gives it
        typedef float f2_t __attribute__((ext_vector_type(2)));
        typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int e = 0; e < E; e += 2) {
            const f2_t prod = {__fmul_rn(code_of(e), scale), __fmul_rn(code_of(e + 1), scale)};
            const uint32_t pb = __builtin_bit_cast(uint32_t, __builtin_convertvector(prod, bf2_t));
            const f2_t sum = {__fadd_rn(__builtin_bit_cast(float, pb << 16), zero), __fadd_rn(__builtin_bit_cast(float, pb & 0xFFFF0000u), zero)};
            uint32_t sb = __builtin_bit_cast(uint32_t, __builtin_convertvector(sum, bf2_t));
            if (sum.x != sum.x) sb = (sb & 0xFFFF0000u) | 0x7FC0u;
            if (sum.y != sum.y) sb = (sb & 0x0000FFFFu) | 0x7FC00000u;
            words[e / 2] = sb;
        }
    } else {
        S out[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float prod = Elem<DT>::load(Elem<DT>::store(__fmul_rn(code_of(e), scale)));
            out[e] = Elem<DT>::store(__fadd_rn(prod, zero));
        }
        if constexpr (sizeof(S) == 2) {
#pragma unroll
            for (int e = 0; e < E; e += 2) words[e / 2] = out[e] | (static_cast<uint32_t>(out[e + 1]) << 16);
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) words[e] = __builtin_bit_cast(uint32_t, out[e]);
        }
    }
    const uint4 v = make_uint4(words[0], words[1], words[2], words[3]);
    *reinterpret_cast<uint4*>(W + static_cast<size_t>(n) * K + kT * 32 + p * E) = v;
}

template <int DT>
void launch_dequantize_rows(const uint4* packed, const void* sz, void* out, int64_t N, int64_t K, int64_t group, hipStream_t s) {
    using S = typename Elem<DT>::storage;
    constexpr int kTilesPerGroup = 32 / (32 / (16 / static_cast<int>(sizeof(S))));
    const int k_super = static_cast<int>(K / 32);
    const int chunks = (k_super + kTilesPerGroup - 1) / kTilesPerGroup;
    int4_dequantize_rows_kernel<DT><<<dim3(static_cast<unsigned>((N / 8) * chunks)), 256, 0, s>>>(
        packed, static_cast<const S*>(sz), static_cast<S*>(out), static_cast<int>(N), static_cast<int>(K), k_super,
        static_cast<int>(group / 32), chunks);
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT size_t tpq_int4_mm_workspace_bytes(int64_t N) {
    // counters + up to 16 slices of 4 rows of fp32 partial columns
    return N <= 0 ? 0 : kCounterBytes + static_cast<size_t>(16) * 4 * static_cast<size_t>(N) * sizeof(float);
}

TPQ_EXPORT size_t tpq_int4_mm_rows_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    // the decode kernels' share, and for 33 .. 256 rows up to 16 slices of fp32 sums for the tiled kernel
    size_t bytes = tpq_int4_mm_workspace_bytes(N);
    if (M >= kInt4GemmRowsSliced && M <= 256 && N > 0 && K >= 128) {
        const int slices = int4_gemm_slices(M, N, K, ~static_cast<size_t>(0));
        const size_t tiled = kCounterBytes + static_cast<size_t>(slices) * static_cast<size_t>(M) * static_cast<size_t>(N) * sizeof(float);
        if (slices > 1 && tiled > bytes) bytes = tiled;
    }
    return bytes;
}

TPQ_EXPORT int tpq_int4_mm_ws(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed,
                              int inner_k_tiles, int64_t N, int64_t group, const void* scales_and_zeros,
                              void* out, void* workspace, size_t workspace_bytes, void* stream) {
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
        if (workspace && !aligned(workspace, 16)) workspace = nullptr;
        if (dtype == TPQ_DTYPE_F16)
            return launch_decode<TPQ_DTYPE_F16>(x, M, packed, scales_and_zeros, out, (int)N, (int)K, (int)group, workspace, workspace_bytes, s);
        return launch_decode<TPQ_DTYPE_BF16>(x, M, packed, scales_and_zeros, out, (int)N, (int)K, (int)group, workspace, workspace_bytes, s);
    }
    switch (dtype) {
        case TPQ_DTYPE_F32: return launch_generic<TPQ_DTYPE_F32>(x, M, packed, scales_and_zeros, out, N, K, group, s);
        case TPQ_DTYPE_F16: return launch_generic<TPQ_DTYPE_F16>(x, M, packed, scales_and_zeros, out, N, K, group, s);
        default: return launch_generic<TPQ_DTYPE_BF16>(x, M, packed, scales_and_zeros, out, N, K, group, s);
    }
}

TPQ_EXPORT int tpq_int4_mm(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed,
                           int inner_k_tiles, int64_t N, int64_t group, const void* scales_and_zeros,
                           void* out, void* stream) {
    return tpq_int4_mm_ws(x, dtype, M, K, packed, inner_k_tiles, N, group, scales_and_zeros, out, nullptr, 0, stream);
}

TPQ_EXPORT int tpq_int4_dequantize(const int32_t* packed, int inner_k_tiles, int64_t N, int64_t K, int64_t group,
                                   const void* scales_and_zeros, int dtype, void* out, void* stream) {
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F32 || dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16, TPQ_ERR_INVALID_TYPE,
                "int4 dequantize: unsupported dtype");
    TPQ_REQUIRE(inner_k_tiles == 2, TPQ_ERR_UNSUPPORTED, "int4 dequantize: only innerKTiles = 2 packed weights are supported");
    TPQ_REQUIRE(group == 32 || group == 64 || group == 128, TPQ_ERR_INVALID_VALUE, "int4 dequantize: qGroupSize must be 32, 64 or 128");
    TPQ_REQUIRE(N >= 0 && K >= 0 && N % 8 == 0, TPQ_ERR_INVALID_VALUE, "int4 dequantize: bad shape");
    if (N == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(packed && scales_and_zeros && out && aligned(packed, 16), TPQ_ERR_INVALID_VALUE, "int4 dequantize: null or unaligned pointer");
    const int64_t k_super = (K + 31) / 32, total = N * k_super;
    const int64_t blocks = (total + 255) / 256;
    const unsigned grid = static_cast<unsigned>(blocks > 65535 * 16 ? 65535 * 16 : blocks);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const auto* pp = reinterpret_cast<const uint4*>(packed);
    const int vec = aligned(out, 16) && K % 8 == 0;  // every row segment of 32 outputs starts 16-byte aligned
    if (vec && K % 32 == 0 && N * K <= 0x7FFFFFFF && (N / 8) * ((K / 32 + 3) / 4) <= 0x7FFFFFFF && aligned(scales_and_zeros, 4)) {
        switch (dtype) {
            case TPQ_DTYPE_F32: launch_dequantize_rows<TPQ_DTYPE_F32>(pp, scales_and_zeros, out, N, K, group, s); break;
            case TPQ_DTYPE_F16: launch_dequantize_rows<TPQ_DTYPE_F16>(pp, scales_and_zeros, out, N, K, group, s); break;
            default: launch_dequantize_rows<TPQ_DTYPE_BF16>(pp, scales_and_zeros, out, N, K, group, s); break;
        }
        return check_launch("tpq_int4_dequantize");
    }
    switch (dtype) {
        case TPQ_DTYPE_F32:
            int4_dequantize_kernel<TPQ_DTYPE_F32><<<grid, 256, 0, s>>>(pp, static_cast<const float*>(scales_and_zeros), static_cast<float*>(out), N, K, k_super, group, total, vec);
            break;
        case TPQ_DTYPE_F16:
            int4_dequantize_kernel<TPQ_DTYPE_F16><<<grid, 256, 0, s>>>(pp, static_cast<const uint16_t*>(scales_and_zeros), static_cast<uint16_t*>(out), N, K, k_super, group, total, vec);
            break;
        default:
            int4_dequantize_kernel<TPQ_DTYPE_BF16><<<grid, 256, 0, s>>>(pp, static_cast<const uint16_t*>(scales_and_zeros), static_cast<uint16_t*>(out), N, K, k_super, group, total, vec);
            break;
    }
    return check_launch("tpq_int4_dequantize");
}

namespace {
// shapes the fused entry points are built for: what the matrix-core decode kernel takes
int check_fused(const char* op, int dtype, int64_t M, int64_t K, int inner_k_tiles, int64_t N, int64_t group) {
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16, TPQ_ERR_UNSUPPORTED, "%s: float16 / bfloat16 activations only", op);
    TPQ_REQUIRE(inner_k_tiles == 2, TPQ_ERR_UNSUPPORTED, "%s: only innerKTiles = 2 packed weights are supported", op);
    TPQ_REQUIRE(group == 128, TPQ_ERR_UNSUPPORTED, "%s: qGroupSize must be 128", op);
    TPQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && N % 8 == 0, TPQ_ERR_INVALID_VALUE, "%s: K dimension does not match packed B", op);
    TPQ_REQUIRE(K % 128 == 0 && N <= 0x7FFFFFF8 && K <= 0x7FFFFFE0, TPQ_ERR_UNSUPPORTED, "%s: K must be a multiple of 128", op);
    return TPQ_OK;
}
}  // namespace

TPQ_EXPORT int tpq_int4_mm_add(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed, int inner_k_tiles,
                               int64_t N, int64_t group, const void* scales_and_zeros, const void* residual, void* out,
                               void* stream) {
    if (int rc = check_fused("tpq_int4_mm_add", dtype, M, K, inner_k_tiles, N, group)) return rc;
    if (M == 0 || N == 0) return TPQ_OK;
    TPQ_REQUIRE(K > 0, TPQ_ERR_UNSUPPORTED, "tpq_int4_mm_add: K = 0 is not built");
    TPQ_REQUIRE(x && packed && scales_and_zeros && residual && out, TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_add: null pointer");
    TPQ_REQUIRE(aligned(x, 16) && aligned(packed, 16) && aligned(scales_and_zeros, 16) && aligned(residual, 8) && aligned(out, 8) && N % 4 == 0,
                TPQ_ERR_UNSUPPORTED, "tpq_int4_mm_add: unaligned operand");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == TPQ_DTYPE_F16)
        return launch_fused<TPQ_DTYPE_F16>(x, M, packed, scales_and_zeros, nullptr, nullptr, residual, out, (int)N, (int)K, (int)group, s);
    return launch_fused<TPQ_DTYPE_BF16>(x, M, packed, scales_and_zeros, nullptr, nullptr, residual, out, (int)N, (int)K, (int)group, s);
}

namespace {
int swiglu_entry(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed_gate, const int32_t* packed_up,
                 int inner_k_tiles, int64_t N, int64_t group, const void* sz_gate, const void* sz_up, void* out, void* stream,
                 const void* norm_weight, float norm_eps);
int multi_entry(const void* x, int dtype, int64_t M, int64_t K, int count, const int32_t* const* packed, int inner_k_tiles,
                const int64_t* N, int64_t group, const void* const* scales_and_zeros, void* const* out, void* stream,
                const void* norm_weight, float norm_eps);
}  // namespace

TPQ_EXPORT int tpq_int4_mm_swiglu(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed_gate,
                                  const int32_t* packed_up, int inner_k_tiles, int64_t N, int64_t group,
                                  const void* sz_gate, const void* sz_up, void* out, void* stream) {
    return swiglu_entry(x, dtype, M, K, packed_gate, packed_up, inner_k_tiles, N, group, sz_gate, sz_up, out, stream, nullptr, 0.0f);
}

TPQ_EXPORT int tpq_int4_mm_swiglu_norm(const void* x, int dtype, int64_t M, int64_t K, const void* norm_weight, float eps,
                                       const int32_t* packed_gate, const int32_t* packed_up, int inner_k_tiles, int64_t N,
                                       int64_t group, const void* sz_gate, const void* sz_up, void* out, void* stream) {
    TPQ_REQUIRE(norm_weight != nullptr && aligned(norm_weight, 16), TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_swiglu_norm: null or unaligned norm weight");
    TPQ_REQUIRE(eps >= 0.0f, TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_swiglu_norm: negative eps");
    return swiglu_entry(x, dtype, M, K, packed_gate, packed_up, inner_k_tiles, N, group, sz_gate, sz_up, out, stream, norm_weight, eps);
}

TPQ_EXPORT int tpq_int4_mm_multi(const void* x, int dtype, int64_t M, int64_t K, int count, const int32_t* const* packed,
                                 int inner_k_tiles, const int64_t* N, int64_t group, const void* const* scales_and_zeros,
                                 void* const* out, void* stream) {
    return multi_entry(x, dtype, M, K, count, packed, inner_k_tiles, N, group, scales_and_zeros, out, stream, nullptr, 0.0f);
}

TPQ_EXPORT int tpq_int4_mm_multi_norm(const void* x, int dtype, int64_t M, int64_t K, const void* norm_weight, float eps, int count,
                                      const int32_t* const* packed, int inner_k_tiles, const int64_t* N, int64_t group,
                                      const void* const* scales_and_zeros, void* const* out, void* stream) {
    TPQ_REQUIRE(norm_weight != nullptr && aligned(norm_weight, 16), TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_multi_norm: null or unaligned norm weight");
    TPQ_REQUIRE(eps >= 0.0f, TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_multi_norm: negative eps");
    return multi_entry(x, dtype, M, K, count, packed, inner_k_tiles, N, group, scales_and_zeros, out, stream, norm_weight, eps);
}

namespace {
int swiglu_entry(const void* x, int dtype, int64_t M, int64_t K, const int32_t* packed_gate, const int32_t* packed_up,
                 int inner_k_tiles, int64_t N, int64_t group, const void* sz_gate, const void* sz_up, void* out, void* stream,
                 const void* norm_weight, float norm_eps) {
    if (int rc = check_fused("tpq_int4_mm_swiglu", dtype, M, K, inner_k_tiles, N, group)) return rc;
    if (M == 0 || N == 0) return TPQ_OK;
    TPQ_REQUIRE(K > 0, TPQ_ERR_UNSUPPORTED, "tpq_int4_mm_swiglu: K = 0 is not built");
    TPQ_REQUIRE(x && packed_gate && packed_up && sz_gate && sz_up && out, TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_swiglu: null pointer");
    TPQ_REQUIRE(aligned(x, 16) && aligned(packed_gate, 16) && aligned(packed_up, 16) && aligned(sz_gate, 16) && aligned(sz_up, 16) &&
                    aligned(out, 8),
                TPQ_ERR_UNSUPPORTED, "tpq_int4_mm_swiglu: unaligned operand");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == TPQ_DTYPE_F16)
        return launch_fused<TPQ_DTYPE_F16>(x, M, packed_gate, sz_gate, packed_up, sz_up, nullptr, out, (int)N, (int)K, (int)group, s, norm_weight, norm_eps);
    return launch_fused<TPQ_DTYPE_BF16>(x, M, packed_gate, sz_gate, packed_up, sz_up, nullptr, out, (int)N, (int)K, (int)group, s, norm_weight, norm_eps);
}

int multi_entry(const void* x, int dtype, int64_t M, int64_t K, int count, const int32_t* const* packed, int inner_k_tiles,
                const int64_t* N, int64_t group, const void* const* scales_and_zeros, void* const* out, void* stream,
                const void* norm_weight, float norm_eps) {
    TPQ_REQUIRE(count >= 1 && count <= kMultiMax, TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_multi: 1 to %d weights per call", kMultiMax);
    TPQ_REQUIRE(packed && N && scales_and_zeros && out, TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_multi: null pointer");
    int64_t n_total = 0;
    for (int w = 0; w < count; ++w) {
        if (int rc = check_fused("tpq_int4_mm_multi", dtype, M, K, inner_k_tiles, N[w], group)) return rc;
        n_total += N[w];
    }
    TPQ_REQUIRE(n_total <= 0x7FFFFFF8, TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_multi: dimension too large");
    if (M == 0 || n_total == 0) return TPQ_OK;
    TPQ_REQUIRE(K > 0, TPQ_ERR_UNSUPPORTED, "tpq_int4_mm_multi: K = 0 is not built");
    TPQ_REQUIRE(x && aligned(x, 16), TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_multi: null or unaligned activations");
    for (int w = 0; w < count; ++w) {
        if (N[w] == 0) continue;
        TPQ_REQUIRE(packed[w] && scales_and_zeros[w] && out[w], TPQ_ERR_INVALID_VALUE, "tpq_int4_mm_multi: null pointer");
        TPQ_REQUIRE(aligned(packed[w], 16) && aligned(scales_and_zeros[w], 16) && aligned(out[w], 8), TPQ_ERR_UNSUPPORTED,
                    "tpq_int4_mm_multi: unaligned operand");
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == TPQ_DTYPE_F16)
        return launch_multi<TPQ_DTYPE_F16>(x, M, count, packed, N, scales_and_zeros, out, (int)K, (int)group, s, norm_weight, norm_eps);
    return launch_multi<TPQ_DTYPE_BF16>(x, M, count, packed, N, scales_and_zeros, out, (int)K, (int)group, s, norm_weight, norm_eps);
}
}  // namespace
