// int4 decode for 2..16 activation rows on the matrix cores, every load of a wavefront in flight at once.
//
// Same arithmetic as int4_mfma_kernel.h (A = unpacked weights, B = activations, one correction MFMA per eight k,
// y += scale (D - corr) + zero sx per step of 128 k).  A workgroup is 16 wavefronts and owns NB blocks of 16 output
// channels; wavefront w owns the steps w, w + 16, ... (at most SPW of them) and requests all of them before it
// looks at the first, in straight-line code.  Three things make that form faster than the loop with two steps in
// flight:
//
//   * Loads return in the order of their requests, and a branch between request and use makes the compiler wait
//     for every outstanding load at the join.  Here the small loads go first (the (scale, zero) words, then the
//     activations, then the weights in the order of their use), nothing branches before the last step, and each
//     step waits for exactly its own weights.
//
//   * The activations reach the lanes through LDS.  The MFMA wants lane (m, q) to hold the 64 bytes
//     x[m][32 (4 s + q) ..] of its row: loaded directly, one 16-byte load per lane touches 32 cache lines per
//     wavefront instruction and uses a quarter of each, four times the line look-ups of a contiguous read, and all
//     16 rows are fetched whatever M is.  Here a wavefront instruction reads four rows x 256 contiguous bytes
//     (8 lines, fully used), only the XR rows that can be live (rows >= M re-read row M - 1), stores them to a
//     wavefront-private LDS tile with rows 272 bytes apart, and each lane reads its 4 x 16 bytes from there
//     (eight rows x 16 bytes cover all banks once; lanes of rows >= XR read row m % XR: their columns of D are
//     never stored).  With direct loads the time followed the number of distinct rows read (4096 -> 11008, fp16,
//     48 channels per workgroup: 7.0 / 7.0 / 7.6 / 8.1 us at 2 / 4 / 8 / 12 rows).
//
//   * The (scale, zero) words travel as one word per lane (lane l = channel l of the workgroup), are parked in
//     LDS and read back as the 16 bytes per block the epilogue wants: SPW registers in flight instead of 4 NB SPW.
//
// A launch serves up to four weights that share the activations (the q, k and v projections of a decoder layer):
// the blocks of 16 channels of all weights are numbered through, and a workgroup takes NB consecutive ones.
// Pair mode: NB / 2 blocks of a gate weight and the same blocks of an up weight; the output is silu_mul(gate, up).
// NORM: y = rms_norm(x, g, eps) . W^T, the norm -> projection pairs of a decoder layer
// (benchmark/bench_llama_e2e.py:113-114, 126-128, 143), with rms_norm(x)[k] = (x[k] * rsqrt(mean(x^2) + eps)) * g[k]
// (tensorplay/nn/functional.py:2350-2372).  The factor rsqrt(...) is one number per row, so it is taken out of the
// sum: the activations are multiplied by g on their way into LDS (rounded to the activation dtype there, where the
// reference rounds the normalized value: the same relative error), every wavefront adds the squares of its steps
// (v_dot2 of the value with itself), and the finishing wavefront multiplies the row's sum by rsqrt(mean + eps) before
// it rounds.  No barrier and no division in front of the products, no launch and no round trip of the activations
// through memory for the norm; every workgroup does it for itself.  Results agree with the reference's two-step
// formulation to the matmul's own tolerance, not bit for bit.
#pragma once

#include "int4_mfma_kernel.h"

namespace tpq {
namespace {

constexpr int kFlightWaves = 16;
constexpr int kFlightRowStride = 272;  // bytes between the rows of an activation tile in LDS (256 + 16)
constexpr int kFlightMaxWeights = 4;
constexpr int kFlightOne = 0, kFlightPair = 1, kFlightMany = 2;  // one weight; gate and up with SwiGLU; two to four weights

// One member per weight, not arrays: selecting among array elements with a wave-uniform index is turned into
// dynamic indexing of the kernel arguments, which moves them to scratch memory.
struct FlightWeight {
    const uint4* packed;
    const uint32_t* sz;
    uint16_t* y;
    int N;
    int first;  // first block (of 16 channels) of the weight in the launch's numbering
};
struct FlightSet {
    FlightWeight w0, w1, w2, w3;
    int count;
    const uint16_t* norm_weight;  // NORM: [K] of the activation dtype
    float norm_eps, norm_inv_k;   // eps and 1 / K
};

// Keeps the memory operations on either side in program order, for the compiler's code motion and for its
// instruction scheduler; no instruction.  Loads through a __restrict__ const pointer are not held by it (nothing
// the fence could do would change what they read): such a pointer goes through opaque4 / opaque1 first.
__device__ __forceinline__ void order_fence() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
typedef const __attribute__((address_space(1))) word4_t* GlobalWords4;
typedef const __attribute__((address_space(1))) uint32_t* GlobalWord;
__device__ __forceinline__ GlobalWords4 opaque4(const void* p) {
    asm volatile("" : "+v"(p));
    return (GlobalWords4)p;  // still a global address, of provenance unknown to the compiler
}
__device__ __forceinline__ GlobalWord opaque1(const void* p) {
    asm volatile("" : "+v"(p));
    return (GlobalWord)p;
}
__device__ __forceinline__ uint4 as_uint4(word4_t v) { return make_uint4(v.x, v.y, v.z, v.w); }
// Workgroup barrier that orders LDS traffic only: __syncthreads() would also wait for every outstanding global load,
// i.e. for the weights that are meant to stay in flight across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// steps of activations resident in LDS per wavefront at a time
template <int XR>
constexpr int flight_resident_steps() { return XR == 16 ? 1 : 2; }

// (the same for one and for two row blocks: the second block reuses the tiles and the partial-sum area of the first)
template <int NB, int SPW, int XR>
constexpr size_t flight_lds_bytes() {
    return static_cast<size_t>(kFlightWaves) * flight_resident_steps<XR>() * XR * kFlightRowStride  // activation tiles
         + static_cast<size_t>(kFlightWaves) * SPW * (NB > 4 ? 2 : 1) * kWave * 4                    // parameter words
         + static_cast<size_t>(kFlightWaves) * NB * 4 * (4 * XR) * 4                                 // partial sums, live rows
         + static_cast<size_t>(kFlightWaves) * XR * 4 * 2;                                           // NORM: sums of squares, and the power of two each row was scaled by
}

// x: [M][K] 16-bit, M <= XR; weights as in FlightSet (packed: [N/8][K/32][8] x 16 bytes; sz: [K/group][N] words
// (scale, zero)); K % 128 == 0, 16 <= K / 128 <= 16 SPW and K / 128 > 16 (SPW - 1); a group is 128 << group_shift k;
// residual (one weight, may be null): [M][N], added to the rounded output.
// RB = 2 (XR = 16, one weight or several, not the pair): 17..32 rows as two blocks of 16.  The weights are requested once and stay in registers;
// the second block's activations are requested step by step into the registers the first block's have left for LDS, and
// are multiplied with the same weights (unpacked again) when the first block is done.
template <int DT, int NB, int SPW, int XR, int MODE, bool NORM = false, int RB = 1>
__global__ __launch_bounds__(kFlightWaves* kWave) void int4_mfma_flight_kernel(const uint16_t* __restrict__ x, FlightSet set, int M,
                                                                              int K, int group_shift,
                                                                              const uint16_t* __restrict__ residual) {
    static_assert(XR == 4 || XR == 8 || XR == 16, "rows through LDS: 4, 8 or 16");
    static_assert(RB == 1 || (RB == 2 && XR == 16 && !NORM && MODE != kFlightPair), "two row blocks: 16 rows each, not for the pair");
    constexpr bool PAIR = MODE == kFlightPair;
    static_assert(!PAIR || NB % 2 == 0, "a pair is the same blocks of two weights");
    static_assert(NB <= 8, "two parameter words per lane at most");
    using L = Lane16<DT>;
    using ML = MfmaLane<DT>;
    constexpr int XS = flight_resident_steps<XR>();
    constexpr int PW = NB > 4 ? 2 : 1;   // parameter words per lane and step
    constexpr int C = PAIR ? NB / 2 : NB;  // output blocks
    extern __shared__ __align__(16) unsigned char flight_lds[];
    unsigned char* const xbuf = flight_lds;
    uint32_t* const par = reinterpret_cast<uint32_t*>(flight_lds + static_cast<size_t>(kFlightWaves) * XS * XR * kFlightRowStride);
    float* const red = reinterpret_cast<float*>(par + kFlightWaves * SPW * PW * kWave);  // [wave][NB][4][4 XR]

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int k_super = K / 32, steps = K / 128;

    // block b of this workgroup: its weight and first channel (wave-uniform); a block past the end of its weight
    // starts at N: loads are clamped to valid addresses, nothing is stored
    struct Block {
        const uint4* packed;
        const uint32_t* sz;
        uint16_t* y;
        int N, n0;
    };
    auto weight_of = [&](int numbered) {  // scalar selects, member by member: no branch, no indexing of the arguments
        Block sel;
        sel.packed = set.w0.packed; sel.sz = set.w0.sz; sel.y = set.w0.y; sel.N = set.w0.N; sel.n0 = set.w0.first;
#define TPQ_PICK(WN, IDX)                                               \
    {                                                                   \
        const bool pick = set.count > IDX && numbered >= set.WN.first;  \
        sel.packed = pick ? set.WN.packed : sel.packed;                 \
        sel.sz = pick ? set.WN.sz : sel.sz;                             \
        sel.y = pick ? set.WN.y : sel.y;                                \
        sel.N = pick ? set.WN.N : sel.N;                                \
        sel.n0 = pick ? set.WN.first : sel.n0;                          \
    }
        TPQ_PICK(w1, 1) TPQ_PICK(w2, 2) TPQ_PICK(w3, 3)
#undef TPQ_PICK
        return sel;  // n0 = first block of the weight
    };
    auto resolve = [&](int b) {
        Block blk;
        int local;
        if constexpr (MODE == kFlightPair) {
            local = static_cast<int>(blockIdx.x) * C + (b >= C ? b - C : b);
            blk.packed = b >= C ? set.w1.packed : set.w0.packed;
            blk.sz = b >= C ? set.w1.sz : set.w0.sz;
            blk.y = set.w0.y; blk.N = set.w0.N;
        } else if constexpr (MODE == kFlightOne) {
            local = static_cast<int>(blockIdx.x) * NB + b;
            blk.packed = set.w0.packed; blk.sz = set.w0.sz; blk.y = set.w0.y; blk.N = set.w0.N;
        } else {
            const int numbered = static_cast<int>(blockIdx.x) * NB + b;
            blk = weight_of(numbered);
            local = numbered - blk.n0;
        }
        const int n0 = 16 * local;
        blk.n0 = n0 < blk.N ? n0 : blk.N;
        return blk;
    };
    Block blk[NB];
    if constexpr (MODE == kFlightMany && NB > 1) {
        // most workgroups lie inside one weight: one selection for all their blocks
        const int numbered = static_cast<int>(blockIdx.x) * NB;
        const Block lo = weight_of(numbered), hi = weight_of(numbered + NB - 1);
        if (lo.packed == hi.packed && lo.n0 == hi.n0) {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                blk[b] = lo;
                const int n0 = 16 * (numbered + b - lo.n0);
                blk[b].n0 = n0 < lo.N ? n0 : lo.N;
            }
        } else {
#pragma unroll
            for (int b = 0; b < NB; ++b) blk[b] = resolve(b);
        }
    } else {
#pragma unroll
        for (int b = 0; b < NB; ++b) blk[b] = resolve(b);
    }

    // this wavefront's steps; a step past the end (last one only) re-reads the wavefront's first step and is not computed
    int step_of[SPW];
#pragma unroll
    for (int j = 0; j < SPW; ++j) {
        const int s = wave + j * kFlightWaves;
        step_of[j] = s < steps ? s : wave;
    }
    const bool last_live = wave + (SPW - 1) * kFlightWaves < steps;

    // ---- requests: parameters, activations, weights --------------------------------------------------------
    uint32_t pw[SPW][PW];
    {
#pragma unroll
        for (int h = 0; h < PW; ++h) {
            const int mine = q + 4 * h;  // block whose channel i this lane fetches
            const uint32_t* src = blk[0].sz;
            int n = blk[0].n0 + i, width = blk[0].N;
#pragma unroll
            for (int b = 1; b < NB; ++b)
                if (mine == b) { src = blk[b].sz; n = blk[b].n0 + i; width = blk[b].N; }
            const GlobalWord p_src = opaque1(src + (n < width ? n : width - 1));
#pragma unroll
            for (int j = 0; j < SPW; ++j) pw[j][h] = p_src[static_cast<size_t>(step_of[j] >> group_shift) * width];
        }
    }
    order_fence();
    uint4 xg[SPW][XR / 4];
#pragma unroll
    for (int t = 0; t < XR / 4; ++t) {
        int row = 4 * t + q;
        row = row < M ? row : M - 1;
        const GlobalWords4 src = opaque4(reinterpret_cast<const uint4*>(x + static_cast<size_t>(row) * K) + i);
#pragma unroll
        for (int j = 0; j < SPW; ++j) xg[j][t] = as_uint4(src[step_of[j] * 16]);
    }
    uint4 gk[NORM ? SPW : 1];  // NORM: the norm weights of this lane's eight k per step
    if constexpr (NORM) {
        const GlobalWords4 src = opaque4(reinterpret_cast<const uint4*>(set.norm_weight) + i);
#pragma unroll
        for (int j = 0; j < SPW; ++j) gk[j] = as_uint4(src[step_of[j] * 16]);
    }
    order_fence();
    uint4 w[SPW][NB];
    {
        GlobalWords4 w_base[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int n_tiles = blk[b].N >> 3;
            int tile = (blk[b].n0 + i) >> 3;
            tile = tile < n_tiles ? tile : n_tiles - 1;  // channels past N: any valid tile, result dropped
            w_base[b] = opaque4(blk[b].packed + (static_cast<size_t>(tile) * k_super + q) * 8 + (i & 7));
        }
#pragma unroll
        for (int j = 0; j < SPW; ++j) {  // in the order of their use: a step waits for its own blocks only
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                w[j][b] = as_uint4(__builtin_nontemporal_load(w_base[b] + static_cast<size_t>(step_of[j]) * 32));
                order_fence();
            }
            if (j == 0 && SPW > 1) {
                // The memory system takes a compute unit's requests oldest wavefront first, at the rate it returns data:
                // without a pause the first wavefronts have asked for all their steps before the last ones have asked
                // for any, and the steps of the last wavefronts arrive together at the end, their arithmetic trailing
                // the stream.  512 clocks let the other wavefronts' first steps go out first (4096 -> 11008 at 8 rows:
                // 6.93 -> 6.79 us; 8192 x 8192: 9.5 -> 9.2; nothing lost elsewhere).
                __builtin_amdgcn_s_sleep(8);
                order_fence();
            }
        }
    }

    // constant A of the correction MFMA: row 0 = offset + 8 of the pair parity, row 1 = ones
    uint32_t a_corr_even = 0, a_corr_odd = 0;
    if (i == 0) { a_corr_even = ML::kOffEven; a_corr_odd = ML::kOffOdd; }
    if (i == 1) { a_corr_even = ML::kOnes; a_corr_odd = ML::kOnes; }
    uint32_t magic_even, magic_odd;  // kept in VGPRs behind an opaque move: v_and_or_b32 takes one literal only
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_even) : "s"(L::kMagicEven));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_odd) : "s"(L::kMagicOdd));

    // ---- the small loads are parked in LDS, wavefront-private: no barrier, the LDS operations of a wavefront keep
    // their order; the activation tiles hold XS steps at a time
    unsigned char* const my_x = xbuf + static_cast<size_t>(wave) * XS * XR * kFlightRowStride;
    uint32_t* const my_par = par + wave * SPW * PW * kWave;
#pragma unroll
    for (int j = 0; j < SPW; ++j)
#pragma unroll
        for (int h = 0; h < PW; ++h) my_par[(j * PW + h) * kWave + lane] = pw[j][h];

    float* const ssq = red + kFlightWaves * NB * 4 * (4 * XR);  // [wave][XR], NORM only
    float* const undo = ssq + kFlightWaves * XR;                // [wave][XR], NORM with fp16: 2^(ex + eg) of the row's products
    if constexpr (NORM) {
        // lane (i, q) holds eight k of row 4 t + q per step: squares added per row, the values multiplied by g in place.
        // The products x g are rounded to the activation type before the row's factor is known.  bfloat16 has float's
        // exponent range.  fp16 does not (x g beyond 65504 would become inf, x g below 6e-5 subnormal), so there both
        // factors are first scaled by exact powers of two taken from bounds this wavefront already has: |x| <= sqrt of
        // its sum of squares of the row, |g| < 2^eg over its k.  The scaled products stay within [-4, 4]; the wavefront's
        // partial sums of the row are multiplied by 2^(ex + eg) again before they leave it.
        const bool last_counts = wave + (SPW - 1) * kFlightWaves < steps;
        [[maybe_unused]] int eg = 0;
        auto pow2_half2 = [](int e) -> uint32_t {  // (2^e, 2^e) as two fp16, e in [-16, 15]
            const uint32_t h = e >= -14 ? static_cast<uint32_t>(e + 15) << 10 : 0x0400u >> (-14 - e);
            return h | (h << 16);
        };
        if constexpr (DT == TPQ_DTYPE_F16) {
            uint32_t mag = 0;
#pragma unroll
            for (int j = 0; j < SPW; ++j) {
                const uint32_t gw[4] = {gk[j].x, gk[j].y, gk[j].z, gk[j].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t a = gw[e] & 0x7FFF7FFFu;
                    const uint32_t lo = a & 0xFFFFu, hi = a >> 16;
                    mag = mag > lo ? mag : lo;
                    mag = mag > hi ? mag : hi;
                }
            }
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) {
                const uint32_t other = __shfl_xor(mag, off, kWave);
                mag = mag > other ? mag : other;
            }
            eg = static_cast<int>(mag >> 10) - 14;  // |g| < 2^eg (biased exponent - 15 + 1)
            eg = eg < -15 ? -15 : eg > 16 ? 16 : eg;
            const half2_t gs = __builtin_bit_cast(half2_t, pow2_half2(-eg));
#pragma unroll
            for (int j = 0; j < SPW; ++j) {
                gk[j].x = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, gk[j].x) * gs);
                gk[j].y = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, gk[j].y) * gs);
                gk[j].z = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, gk[j].z) * gs);
                gk[j].w = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, gk[j].w) * gs);
            }
        }
#pragma unroll
        for (int t = 0; t < XR / 4; ++t) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < SPW; ++j) {
                const uint32_t xw[4] = {xg[j][t].x, xg[j][t].y, xg[j][t].z, xg[j][t].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (j < SPW - 1 || last_counts) acc = L::dot(xw[e], xw[e], acc);  // a step past the end was read twice
            }
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) acc += __shfl_xor(acc, off, kWave);
            if (i == 0) ssq[wave * XR + 4 * t + q] = acc;  // read behind the barrier at the end
            [[maybe_unused]] half2_t xs;
            if constexpr (DT == TPQ_DTYPE_F16) {
                const int fl = static_cast<int>(__builtin_bit_cast(uint32_t, acc) >> 23) - 127;  // acc >= 0: floor(log2), -127 for 0
                int ex = (fl + 2) >> 1;                                                               // sqrt(acc) < 2^ex
                ex = ex < -15 ? -15 : ex > 16 ? 16 : ex;
                xs = __builtin_bit_cast(half2_t, pow2_half2(-ex));
                if (i == 0) undo[wave * XR + 4 * t + q] = __builtin_bit_cast(float, static_cast<uint32_t>(127 + ex + eg) << 23);
            }
#pragma unroll
            for (int j = 0; j < SPW; ++j) {
                const uint32_t gw[4] = {gk[j].x, gk[j].y, gk[j].z, gk[j].w};
                uint32_t xw[4] = {xg[j][t].x, xg[j][t].y, xg[j][t].z, xg[j][t].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if constexpr (DT == TPQ_DTYPE_F16) {
                        xw[e] = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(half2_t, xw[e]) * xs) * __builtin_bit_cast(half2_t, gw[e]));
                    } else {
                        const float lo = __fmul_rn(bf16_bits_to_f32(static_cast<uint16_t>(xw[e] & 0xFFFFu)), bf16_bits_to_f32(static_cast<uint16_t>(gw[e] & 0xFFFFu)));
                        const float hi = __fmul_rn(bf16_bits_to_f32(static_cast<uint16_t>(xw[e] >> 16)), bf16_bits_to_f32(static_cast<uint16_t>(gw[e] >> 16)));
                        xw[e] = static_cast<uint32_t>(f32_to_bf16_bits(lo)) | (static_cast<uint32_t>(f32_to_bf16_bits(hi)) << 16);
                    }
                }
                xg[j][t] = make_uint4(xw[0], xw[1], xw[2], xw[3]);
            }
        }
    }

    float yacc[RB][NB][4];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) yacc[rb][b][v] = 0.0f;

    auto compute = [&](int j, int rb) {
        // lane (m, q): the 64 bytes of row m % XR in k-tile 4 s + q; MFMA u takes bytes 16 u .. 16 u + 15 of them
        word4_t xb[4];
        const unsigned char* xrow = my_x + ((j % XS) * XR + (i & (XR - 1))) * kFlightRowStride + q * 64;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint4 v = *reinterpret_cast<const uint4*>(xrow + u * 16);
            xb[u] = word4_t{v.x, v.y, v.z, v.w};
        }
        float4_t aux = {0.0f, 0.0f, 0.0f, 0.0f};
        float4_t d[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) d[b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t off = (u & 1) ? a_corr_odd : a_corr_even;
            aux = ML::mfma(word4_t{off, off, off, off}, xb[u], aux);
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            // the weights enter the step here, not earlier: without this the compiler unpacks every block of every
            // step ahead of the first LDS store, which makes the first step wait for the last load
            asm volatile("" : "+v"(w[j][b].x), "+v"(w[j][b].y), "+v"(w[j][b].z), "+v"(w[j][b].w)::"memory");
            uint32_t v[4][4];  // [word r][pair u] = codes at k = 2 r + 8 u, + 1 of the lane's k-tile
#pragma unroll
            for (int r = 0; r < 4; ++r) L::template unpack<true>(dword_of(w[j][b], r), v[r], magic_even, magic_odd);
#pragma unroll
            for (int u = 0; u < 4; ++u) d[b] = ML::mfma(word4_t{v[0][u], v[1][u], v[2][u], v[3][u]}, xb[u], d[b]);
        }
        // rows 0 and 1 of the correction product sit in lanes 0..15, registers 0 and 1
        const float corr = __shfl(aux[0], i, kWave), sx = __shfl(aux[1], i, kWave);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint4 p = *reinterpret_cast<const uint4*>(my_par + j * PW * kWave + 16 * b + 4 * q);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t word = dword_of(p, v);  // (scale, zero) of channel n0 + 4 q + v of block b
                yacc[rb][b][v] = __builtin_fmaf(L::lo(word), d[b][v] - corr, __builtin_fmaf(L::hi(word), sx, yacc[rb][b][v]));
            }
        }
    };

#pragma unroll
    for (int j0 = 0; j0 < SPW; j0 += XS) {
#pragma unroll
        for (int j = j0; j < j0 + XS && j < SPW; ++j)
#pragma unroll
            for (int t = 0; t < XR / 4; ++t)
                *reinterpret_cast<uint4*>(my_x + ((j % XS) * XR + 4 * t + q) * kFlightRowStride + i * 16) = xg[j][t];
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (RB == 2) {  // XS = 1: step j0 of the first block is in LDS, its registers take the second block's
            order_fence();
#pragma unroll
            for (int t = 0; t < XR / 4; ++t) {
                int row = XR + 4 * t + q;
                row = row < M ? row : M - 1;
                const GlobalWords4 src = opaque4(reinterpret_cast<const uint4*>(x + static_cast<size_t>(row) * K) + i);
                xg[j0][t] = as_uint4(src[step_of[j0] * 16]);
            }
            order_fence();
        }
#pragma unroll
        for (int j = j0; j < j0 + XS && j < SPW; ++j) {
            if (j < SPW - 1) {
                compute(j, 0);
            } else if (last_live) {  // wave-uniform, after every request: nothing is held back by this branch
                compute(j, 0);
            }
            __builtin_amdgcn_sched_barrier(0);  // a step is finished, epilogue included, while the next one is on its way
        }
        __builtin_amdgcn_wave_barrier();
    }
    if constexpr (RB == 2) {
        static_assert(RB == 1 || XS == 1, "the second block's requests go step by step");
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
#pragma unroll
            for (int t = 0; t < XR / 4; ++t) *reinterpret_cast<uint4*>(my_x + (4 * t + q) * kFlightRowStride + i * 16) = xg[j][t];
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_sched_barrier(0);
            if (j < SPW - 1) {
                compute(j, 1);
            } else if (last_live) {
                compute(j, 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_wave_barrier();
        }
    }

    // ---- the wavefronts' partial sums, added in wavefront order -----------------------------------------------
    const int slot = q * XR + i;  // live lanes (rows < XR) only
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
    if (rb > 0) __syncthreads();  // the sums of the first block have been read
    if (i < XR) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float part = yacc[rb][b][v];
                if constexpr (NORM && DT == TPQ_DTYPE_F16) part *= undo[wave * XR + i];  // this wavefront's own write, same row: exact
                red[((wave * NB + b) * 4 + v) * (4 * XR) + slot] = part;
            }
    }
    __syncthreads();
    const int out_row = XR * rb + i;  // RB = 1: i
    // wavefront w finishes output block w: lane (m, q) stores row m, channels n0 + 4 q + v
    for (int b = wave; b < C; b += kFlightWaves) {
        if (i >= XR || out_row >= M) continue;
        const Block out = resolve(b);
        const int n = out.n0 + 4 * q;
        if (n >= out.N) continue;  // N % 8 == 0 and n % 4 == 0: all four channels exist
        float sum[PAIR ? 2 : 1][4];
#pragma unroll
        for (int h = 0; h < (PAIR ? 2 : 1); ++h)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                sum[h][v] = 0.0f;
#pragma unroll
                for (int ww = 0; ww < kFlightWaves; ++ww) sum[h][v] += red[((ww * NB + b + h * C) * 4 + v) * (4 * XR) + slot];
            }
        if constexpr (NORM) {  // the row's factor rsqrt(mean(x^2) + eps)
            float total = 0.0f;
#pragma unroll
            for (int ww = 0; ww < kFlightWaves; ++ww) total += ssq[ww * XR + i];
            const float inv = __builtin_amdgcn_rsqf(__builtin_fmaf(total, set.norm_inv_k, set.norm_eps));
#pragma unroll
            for (int h = 0; h < (PAIR ? 2 : 1); ++h)
#pragma unroll
                for (int v = 0; v < 4; ++v) sum[h][v] *= inv;
        }
        uint16_t o[4];
        if constexpr (PAIR) {
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = swiglu_of<DT>(sum[0][v], sum[1][v]);
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = L::out(sum[0][v]);
            if (residual != nullptr) {  // the rounded output plus the residual, rounded again: what a separate add does
                const uint2 rw = *reinterpret_cast<const uint2*>(residual + static_cast<size_t>(out_row) * out.N + n);
                const uint16_t rv[4] = {static_cast<uint16_t>(rw.x), static_cast<uint16_t>(rw.x >> 16), static_cast<uint16_t>(rw.y),
                                        static_cast<uint16_t>(rw.y >> 16)};
#pragma unroll
                for (int v = 0; v < 4; ++v) o[v] = L::out(Elem<DT>::load(o[v]) + Elem<DT>::load(rv[v]));
            }
        }
        *reinterpret_cast<uint2*>(out.y + static_cast<size_t>(out_row) * out.N + n) =
            make_uint2(o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16));
    }
    }
}

}  // namespace
}  // namespace tpq
