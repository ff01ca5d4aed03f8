// int4 decode kernel for 1..16 (MB = 2: ..32) activation rows on the matrix cores (fp16 / bf16,
// group a multiple of 128, K % 128 == 0): every packed byte is read once for
// all rows, and the multiply-accumulate work leaves the vector ALU.
//
// v_mfma_f32_16x16x32 computes D[i][j] += sum_k A[i][k] B[k][j] with lane
// l = (i or j) + 16 q holding the eight k-slots 8q..8q+7 of its row / column.
// Which actual k sits in a slot is free as long as A and B agree, and that is
// what makes the packed layout usable without any shuffle:
//   * A = weights.  Lane (i, q) owns row n0 + i and, in a step of four k-tiles
//     (128 k), the k-tile 4 s + q: one 16-byte load = the row's four words =
//     all 32 k of that tile.  A word unpacks in place into four 16-bit pairs
//     (magic + code, see int4_lane.h); pair j of word r is k = 2r + 8j, + 1, and
//     pair j of the four words is the A operand of MFMA j: four MFMAs per step
//     and 16 rows.
//   * B = activations.  Lane (m, q) loads the 64 bytes x[m][32 (4s+q) .. +32)
//     and the operand of MFMA j is simply dwords 4j .. 4j+3 of them (k = 8j ..
//     8j+7, the same eight k as the weight pairs), one 16-byte load.  Columns
//     m >= M stay zero and are dropped.
//   * One more MFMA per eight k with a constant A (row 0: the magic offsets + 8,
//     row 1: ones) yields, per activation row, corr = sum x (offset + 8) and
//     sx = sum x over the step; they come out in lanes 0..15 and are broadcast
//     with two cross-lane reads.
//   * D is lane (m, q) x rows n0 + 4q + v.  A step lies inside one quantization
//     group, so after its MFMAs  y += scale (D - corr) + zero sx  in fp32 with
//     this lane's four (scale, zero) pairs, one 16-byte load.
// A workgroup owns 16 NB consecutive output channels; its wavefronts take the
// steps round-robin and meet in LDS at the end.
#pragma once

#include "int4_lane.h"

namespace tpq {
namespace {


// dword r of a 16-byte vector; r is a constant once the loops around the call are unrolled
__device__ __forceinline__ uint32_t dword_of(const uint4& q, int r) { return r == 0 ? q.x : r == 1 ? q.y : r == 2 ? q.z : q.w; }

typedef uint32_t word4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));

template <int DT>
struct MfmaLane;
template <>
struct MfmaLane<TPQ_DTYPE_F16> {
    static constexpr uint32_t kOffEven = 0x64086408u, kOffOdd = 0x54805480u, kOnes = 0x3C003C00u;  // 1032, 72, 1
    static __device__ __forceinline__ float4_t mfma(const word4_t& a, const word4_t& b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    }
};
template <>
struct MfmaLane<TPQ_DTYPE_BF16> {
    static constexpr uint32_t kOffEven = 0x43084308u, kOffOdd = 0x43084308u, kOnes = 0x3F803F80u;  // 136, 136, 1
    static __device__ __forceinline__ float4_t mfma(const word4_t& a, const word4_t& b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, a), __builtin_bit_cast(bf8_t, b), c, 0, 0, 0);
    }
};

// SwiGLU gate of two rounded outputs, as the unfused sequence computes it: silu_mul on the 16-bit
// results in fp32, gate * sigmoid(gate) * up, rounded once (reference: silu_mul_loop,
// p10/src/backend/cpu/PointwiseKernels.cpp:1466-1478).
template <int DT>
__device__ __forceinline__ uint16_t swiglu_of(float gate_sum, float up_sum) {
    using L = Lane16<DT>;
    const float g = Elem<DT>::load(L::out(gate_sum)), u = Elem<DT>::load(L::out(up_sum));
    const float sigmoid = __fdiv_rn(1.0f, 1.0f + expf(-g));
    return L::out(g * sigmoid * u);
}

// x: [M][K] 16-bit; packed: [N/8][K/32][8] x 16 bytes; sz: [K/group][N] words (scale, zero);
// steps = K / 128; a group is 128 << group_shift k.
// PAIR (NB = 2): the two blocks are the same 16 channels of two weights (packed / sz: gate, packed_b /
// sz_b: up) and the output is silu_mul(gate, up).  residual (plain mode, may be null): [M][N], added to
// the rounded output.
// GKT = k-tiles (of 32) per quantization group: 4 stands for groups of 128 k and more (above).  Groups of 32
// or 64 k (GKT = 1, 2) differ between the four lanes an MFMA adds up, so there the weights are dequantized in
// registers before the product, no offset MFMA, no per-step epilogue.  fp16: the packed fp16 operations and
// roundings of the reference's own dense weight, T(code - 8) * scale + zero (int4_tc_dequantize_kernel,
// QuantGemmKernels.cu:1170-1202), three packed operations per pair.  bf16 (no packed bf16 arithmetic): one fp32
// fma per code and one rounding to bf16, five operations per pair.
// MB = blocks of 16 activation rows per launch (1 or 2): the unpacked weights of a step feed MB column blocks.
// block: index of the workgroup among those of this weight (the grid index when a launch serves one weight).
template <int DT, int NB, int WAVES, bool PAIR = false, int GKT = 4, int MB = 1>
__device__ __forceinline__ void int4_mfma_body(
    const uint16_t* __restrict__ x, const uint4* __restrict__ packed, const uint32_t* __restrict__ sz,
    uint16_t* __restrict__ y, int M, int N, int K, int group_shift, const uint4* __restrict__ packed_b,
    const uint32_t* __restrict__ sz_b, const uint16_t* __restrict__ residual, int block) {
    static_assert(!PAIR || NB == 2, "a pair is two blocks");
    static_assert(GKT == 4 || !PAIR, "in-register dequantization is not built for the pair");
    static_assert(MB == 1 || !PAIR, "the pair takes 16 rows");
    constexpr bool DEQ = GKT < 4;
    using L = Lane16<DT>;
    using ML = MfmaLane<DT>;
    // The activations of a step (256 bytes = two cache lines per row) are read as they lie, four rows = eight whole
    // lines per wave-level load, and reach the MFMA's lanes (lane (m, q): 64 bytes of row m) through a wave-private
    // LDS area, one block of 16 rows at a time, rows 272 bytes apart: asked for in MFMA order every load touches two
    // lines of every row, and the vector memory path charges a load by the lines it touches.  Columns m >= M hold
    // whatever is there; their sums are dropped.  One LDS area serves both uses: the exchange during the steps, the
    // partial sums behind a barrier after them.
    constexpr int kXPitch = 272, kXBytes = 16 * kXPitch;
    constexpr size_t kRedBytes = sizeof(float) * WAVES * NB * MB * 4 * kWave, kXchBytes = static_cast<size_t>(WAVES) * kXBytes;
    __shared__ __align__(16) unsigned char lds_raw[kRedBytes > kXchBytes ? kRedBytes : kXchBytes];
    float (*const red)[NB * MB][4][kWave] = reinterpret_cast<float (*)[NB * MB][4][kWave]>(lds_raw);

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int k_super = K / 32, steps = K / 128, n_tiles = N / 8;
    const int n0 = block * (PAIR ? 16 : 16 * NB);

    // per-lane bases
    const uint4* w_base[NB];
    const uint32_t* sz_base[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int nb0 = PAIR ? n0 : n0 + 16 * b;           // first channel of block b
        int tile = (nb0 + i) >> 3;                         // tile of row nb0 + i
        tile = tile < n_tiles ? tile : n_tiles - 1;        // rows past N: any valid tile, result dropped
        w_base[b] = (PAIR && b == 1 ? packed_b : packed) + (static_cast<size_t>(tile) * k_super + q) * 8 + (i & 7);
        int n4 = nb0 + 4 * q;                              // this lane's four output channels
        n4 = n4 + 4 <= N ? n4 : N - 4;
        sz_base[b] = (PAIR && b == 1 ? sz_b : sz) + n4;
        if constexpr (DEQ) sz_base[b] = sz + ((nb0 + i) < N ? nb0 + i : N - 1);  // (scale, zero) of this lane's weight row
    }
    bool row_live[MB];
#pragma unroll
    for (int r = 0; r < MB; ++r) row_live[r] = 16 * r + i < M;
    // load j of a step: row 4 j + lane / 16, piece lane % 16 of the step's 256 bytes (rows past M: row 0, dropped)
    const uint4* x_base[4 * MB];
#pragma unroll
    for (int j = 0; j < 4 * MB; ++j) {
        const int row = 4 * j + (lane >> 4);
        x_base[j] = reinterpret_cast<const uint4*>(x + static_cast<size_t>(row < M ? row : 0) * K) + (lane & 15);
    }
    unsigned char* const xch_put = lds_raw + wave * kXBytes + (lane >> 4) * kXPitch + (lane & 15) * 16;  // + 4 c rows
    const unsigned char* const xch_get = lds_raw + wave * kXBytes + i * kXPitch + q * 64;                 // + 16 c

    // constant A of the correction MFMA: row 0 = offset + 8 of the pair parity, row 1 = ones
    uint32_t a_corr_even = 0, a_corr_odd = 0;
    if (i == 0) { a_corr_even = ML::kOffEven; a_corr_odd = ML::kOffOdd; }
    if (i == 1) { a_corr_even = ML::kOnes; a_corr_odd = ML::kOnes; }
    uint32_t magic_even, magic_odd;  // kept in VGPRs behind an opaque move: v_and_or_b32 takes one literal only
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_even) : "s"(L::kMagicEven));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_odd) : "s"(L::kMagicOdd));

    struct Step {
        uint4 w[NB];
        uint4 p[NB];
        uint4 xv[MB][4];
    };
    auto load = [&](int s, Step& st) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            st.w[b] = nt_load(w_base[b] + static_cast<size_t>(s) * 32);             // four k-tiles further per step
            // (the whole vector is assigned: writing one member left the steps in scratch memory)
            if constexpr (DEQ) st.p[b] = make_uint4(sz_base[b][static_cast<size_t>((4 * s + q) / GKT) * N], 0u, 0u, 0u);  // group of k-tile 4 s + q
            else st.p[b] = *reinterpret_cast<const uint4*>(sz_base[b] + static_cast<size_t>(s >> group_shift) * N);
        }
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) st.xv[r][c] = x_base[4 * r + c][s * 16];  // as loaded: rows 16 r + 4 c .. + 3
    };

    float yacc[NB][MB][4];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) yacc[b][r][v] = 0.0f;

    auto compute = [&](const Step& st) {
        // the correction product and the weight products alternate, so that no MFMA waits for
        // the one issued just before it
        float4_t aux[MB];
        float4_t d[NB][MB];
#pragma unroll
        for (int r = 0; r < MB; ++r) {
            aux[r] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int b = 0; b < NB; ++b) d[b][r] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
        // each block of 16 rows into the exchange area and this lane's four pieces out of it (LDS keeps a wavefront's
        // accesses in order: the reads of the block before are served before these writes)
        uint4 xq[MB][4];
#pragma unroll
        for (int r = 0; r < MB; ++r) {
#pragma unroll
            for (int c = 0; c < 4; ++c) *reinterpret_cast<uint4*>(xch_put + c * 4 * kXPitch) = st.xv[r][c];
#pragma unroll
            for (int c = 0; c < 4; ++c) xq[r][c] = *reinterpret_cast<const uint4*>(xch_get + c * 16);
        }
        uint32_t v[NB][4][4];  // [block][word r][pair j] = codes at k = 2 r + 8 j, + 1 of the lane's k-tile
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) L::template unpack<true>(dword_of(st.w[b], r), v[b][r], magic_even, magic_odd);
        if constexpr (DEQ && DT == TPQ_DTYPE_BF16) {
            // a pair is (128 + code) twice in bf16: widen both halves (a shift, a mask), one fp32 fma each with
            // zero - 136 scale folded into the addend, and one v_cvt_pk_bf16_f32 back: round-to-nearest-even once
            typedef float f2_t __attribute__((ext_vector_type(2)));
            typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint32_t pw = st.p[b].x;  // (scale, zero) of the lane's row and k-tile
                const float sc = L::lo(pw), zc = __builtin_fmaf(-136.0f, sc, L::hi(pw));
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t pv = v[b][r][j];
                        const f2_t f = {__builtin_fmaf(__builtin_bit_cast(float, pv << 16), sc, zc),
                                        __builtin_fmaf(__builtin_bit_cast(float, pv & 0xFFFF0000u), sc, zc)};
                        v[b][r][j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf2_t));
                    }
            }
        }
        if constexpr (DEQ && DT == TPQ_DTYPE_F16) {
            const half2_t off_even = {static_cast<_Float16>(1032.0f), static_cast<_Float16>(1032.0f)};  // magic + 8
            const half2_t off_odd = {static_cast<_Float16>(72.0f), static_cast<_Float16>(72.0f)};
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint32_t pw = st.p[b].x;  // (scale, zero) of the lane's row and k-tile
                const half2_t s2 = __builtin_bit_cast(half2_t, (pw & 0xFFFFu) | (pw << 16));
                const half2_t z2 = __builtin_bit_cast(half2_t, (pw >> 16) | (pw & 0xFFFF0000u));
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const half2_t code = __builtin_bit_cast(half2_t, v[b][r][j]) - ((j & 1) ? off_odd : off_even);  // exact
                        v[b][r][j] = __builtin_bit_cast(uint32_t, code * s2 + z2);  // rounded after the product and after the sum
                    }
            }
        }
        // MFMA u (16x16x32) covers pair u of the four words of the lane's k-tile: k = 2 r + 8 u, + 1 for
        // r = 0..3, which are dwords 4u .. 4u+3 of the activations, one 16-byte load.
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t off = (u & 1) ? a_corr_odd : a_corr_even;
            word4_t xb[MB];
#pragma unroll
            for (int r = 0; r < MB; ++r) xb[r] = word4_t{xq[r][u].x, xq[r][u].y, xq[r][u].z, xq[r][u].w};
            const word4_t ac = {off, off, off, off};
            if constexpr (!DEQ) {
#pragma unroll
                for (int r = 0; r < MB; ++r) aux[r] = ML::mfma(ac, xb[r], aux[r]);
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const word4_t aw = {v[b][0][u], v[b][1][u], v[b][2][u], v[b][3][u]};
#pragma unroll
                for (int r = 0; r < MB; ++r) d[b][r] = ML::mfma(aw, xb[r], d[b][r]);
            }
        }
        if constexpr (DEQ) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int r = 0; r < MB; ++r)
#pragma unroll
                    for (int v = 0; v < 4; ++v) yacc[b][r][v] += d[b][r][v];
            return;
        }
#pragma unroll
        for (int r = 0; r < MB; ++r) {
            // rows 0 and 1 of the correction product sit in lanes 0..15, registers 0 and 1
            const float corr = __shfl(aux[r][0], i, kWave), sx = __shfl(aux[r][1], i, kWave);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const uint32_t pw = dword_of(st.p[b], v);  // (scale, zero) of channel n0 + 16 b + 4 q + v
                    yacc[b][r][v] = __builtin_fmaf(L::lo(pw), d[b][r][v] - corr, __builtin_fmaf(L::hi(pw), sx, yacc[b][r][v]));
                }
            }
        }
    };

    // this wavefront's steps: wave, wave + WAVES, ...; two in flight (waiting for the prologue's loads in front of the loop,
    // which makes the waits inside it exact, changed nothing here: 4096 x 4096, groups of 64, 8 rows 5.5 -> 5.7 us)
    Step s0 = {}, s1 = {};
    int s = wave;
    if (s < steps) load(s, s0);
    if (s + WAVES < steps) load(s + WAVES, s1);
    for (; s + 3 * WAVES < steps; s += 2 * WAVES) {  // steady state: no branches in the body
        compute(s0);
        load(s + 2 * WAVES, s0);
        compute(s1);
        load(s + 3 * WAVES, s1);
    }
    if (s < steps) {
        compute(s0);
        if (s + 2 * WAVES < steps) load(s + 2 * WAVES, s0);
        if (s + WAVES < steps) compute(s1);
        if (s + 2 * WAVES < steps) compute(s0);
    }

    __syncthreads();  // every wavefront is done with its exchange area
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][b * MB + r][v][lane] = yacc[b][r][v];
    __syncthreads();
    if constexpr (PAIR) {
        if (wave == 0) {  // lane (m, q): channels n0 + 4 q + v of both weights
            float sum[2][4];
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    sum[b][v] = 0.0f;
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) sum[b][v] += red[w][b][v][lane];
                }
            const int n = n0 + 4 * q;
            if (row_live[0] && n < N) {
                const uint32_t lo = swiglu_of<DT>(sum[0][0], sum[1][0]) | (static_cast<uint32_t>(swiglu_of<DT>(sum[0][1], sum[1][1])) << 16);
                const uint32_t hi = swiglu_of<DT>(sum[0][2], sum[1][2]) | (static_cast<uint32_t>(swiglu_of<DT>(sum[0][3], sum[1][3])) << 16);
                *reinterpret_cast<uint2*>(y + static_cast<size_t>(i) * N + n) = make_uint2(lo, hi);
            }
        }
        return;
    }
    // wavefront w finishes output block w, w + W, ... (block = channel block b x row block r): lane (m, q) stores
    // row 16 r + m, channels n0 + 16 b + 4 q + v
    for (int blk = wave; blk < NB * MB; blk += WAVES) {
        const int b = blk / MB, r = blk % MB;
        float sum[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            sum[v] = 0.0f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) sum[v] += red[w][blk][v][lane];
        }
        const int n = n0 + 16 * b + 4 * q;
        const int row = 16 * r + i;
        if (row < M && n < N) {  // N % 8 == 0 and n % 4 == 0: all four channels exist
            uint16_t o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = L::out(sum[v]);
            if (residual != nullptr) {  // the rounded output plus the residual, rounded again: what a separate add does
                const uint2 rw = *reinterpret_cast<const uint2*>(residual + static_cast<size_t>(row) * N + n);
                const uint16_t rv[4] = {static_cast<uint16_t>(rw.x), static_cast<uint16_t>(rw.x >> 16), static_cast<uint16_t>(rw.y),
                                        static_cast<uint16_t>(rw.y >> 16)};
#pragma unroll
                for (int v = 0; v < 4; ++v) o[v] = L::out(Elem<DT>::load(o[v]) + Elem<DT>::load(rv[v]));
            }
            *reinterpret_cast<uint2*>(y + static_cast<size_t>(row) * N + n) =
                make_uint2(o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16));
        }
    }
}

template <int DT, int NB, int WAVES, bool PAIR = false, int GKT = 4, int MB = 1>
__global__ __launch_bounds__(WAVES * kWave) void int4_mfma_kernel(
    const uint16_t* __restrict__ x, const uint4* __restrict__ packed, const uint32_t* __restrict__ sz,
    uint16_t* __restrict__ y, int M, int N, int K, int group_shift, const uint4* __restrict__ packed_b,
    const uint32_t* __restrict__ sz_b, const uint16_t* __restrict__ residual) {
    int4_mfma_body<DT, NB, WAVES, PAIR, GKT, MB>(x, packed, sz, y, M, N, K, group_shift, packed_b, sz_b, residual,
                                                 static_cast<int>(blockIdx.x));
}

// Several weights that share the activations (the q, k and v projections of a decoder layer) in one launch: the
// workgroups of weight w are blocks first[w] .. first[w + 1] - 1 of the grid.  One launch instead of `count` saves
// the launch gap and the ramp of every launch after the first: 4096 x 4096 weights are 8.4 MB each, of whose 5 us
// per launch at most 1.5 us is transfer time.
constexpr int kMultiMax = 4;
struct Int4MultiSet {
    const uint4* packed[kMultiMax];
    const uint32_t* sz[kMultiMax];
    uint16_t* y[kMultiMax];
    int N[kMultiMax];
    int first[kMultiMax + 1];
    int count;
};

template <int DT, int NB, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void int4_mfma_multi_kernel(const uint16_t* __restrict__ x, Int4MultiSet set, int M,
                                                                       int K, int group_shift) {
    const int block = static_cast<int>(blockIdx.x);
    int w = 0;
#pragma unroll
    for (int i = 1; i < kMultiMax; ++i)
        if (i < set.count && block >= set.first[i]) w = i;
    // selected with wave-uniform compares: the struct stays in scalar registers
    const uint4* packed = set.packed[0];
    const uint32_t* sz = set.sz[0];
    uint16_t* y = set.y[0];
    int N = set.N[0], first = set.first[0];
#pragma unroll
    for (int i = 1; i < kMultiMax; ++i)
        if (w == i) { packed = set.packed[i]; sz = set.sz[i]; y = set.y[i]; N = set.N[i]; first = set.first[i]; }
    int4_mfma_body<DT, NB, WAVES>(x, packed, sz, y, M, N, K, group_shift, nullptr, nullptr, nullptr, block - first);
}

}  // namespace
}  // namespace tpq
