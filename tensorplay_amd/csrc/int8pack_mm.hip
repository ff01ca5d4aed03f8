// int8 weight-only matmul: out[m,n] = (sum_k x[m,k] * w[n,k]) * scale[n], out dtype = x dtype
// (reference: _weight_int8pack_mm, p10/src/backend/cuda/QuantGemmKernels.cu:86-180, 339-405:
// activations converted to fp32, fp32 accumulation, per-row scale applied to the sum).
//
// Decode kernel (fp16 / bf16 activations, K % 128 == 0, 1..16 rows per launch), bandwidth bound at one byte
// per weight: v_mfma_f32_16x16x32_f16 with the weights as A and the activations as B, as in the int4
// decode kernel for several rows (NB blocks of 16 channels and 4 or 8 wavefronts per workgroup, chosen by N).
// Lane (i, q) owns weight row n0 + i and, in a step of 128 k, the 32
// bytes at k = 128 s + 32 q: two 16-byte loads, whole 128-byte lines per row and step.  Every dword
// (four int8) becomes two fp16 pairs: xor 0x80808080 turns the bytes into b + 128, v_perm_b32 drops
// each next to the exponent byte 0x64 (fp16 1024 + 128 + b), and one packed fp16 subtract of 1152
// leaves b exactly (bf16: a sign-extending byte-to-float conversion per code, upper halves packed by
// v_perm_b32).  The products are exact and accumulate in fp32 over the whole K range, two
// accumulators taking turns; the per-row scale multiplies the final sum.
//
// Everything else (bf16 / fp32 activations, other K) takes the vector kernel below (wavefront = four channels,
// eight k per lane and turn, fp32 fma), and K % 8 != 0 or unaligned pointers a plain one: one workgroup per
// output channel and slab of up to 8 rows, block reduction.
#include <cstdlib>

#include "int4_flight.h"
#include "int4_lane.h"

namespace tpq {
namespace {

constexpr int kI8Ring = 2;  // steps in flight per wavefront

typedef uint32_t word4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

__device__ __forceinline__ uint32_t dword_at(const uint4& q, int r) { return r == 0 ? q.x : r == 1 ? q.y : r == 2 ? q.z : q.w; }

typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));

// x: [M][K] fp16 or bf16; w: [N][K] int8; scale: [N] fp32; steps = K / 128; NB blocks of 16 channels and MB blocks
// of 16 activation rows per workgroup (the converted weights of a step feed every row block)
//
// The activations of a step are 256 bytes = two cache lines per row.  Asked for in the MFMA's order (lane (m, q): 16
// bytes at 64 q + 16 c of row m, four loads) every load touches two lines of every row, and the vector memory path
// charges a load by the lines it touches: at 32 rows that is 256 line look-ups per step against 16 for the weights.  So
// a wavefront reads them as they lie (lane l: piece l % 16 of row l / 16, four rows = eight whole lines per load) and
// passes them to the MFMA's lanes through a wave-private LDS area, one block of 16 rows at a time (rows 272 bytes apart,
// so that the sixteen rows of a 16-byte read spread over the banks).  Columns m >= M hold whatever is there; their sums
// are dropped.
constexpr int kI8pXPitch = 272;
constexpr int kI8pXBytes = 16 * kI8pXPitch;  // per wavefront

template <int DT, int NB, int MB, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void int8pack_mfma_kernel(
    const uint16_t* __restrict__ x, const int8_t* __restrict__ w, const float* __restrict__ scale,
    uint16_t* __restrict__ y, int M, int N, int K) {
    // one LDS area for both uses: the exchange areas during the steps, the partial sums behind a barrier after them
    constexpr size_t kRedBytes = sizeof(float) * WAVES * NB * MB * 4 * kWave, kXchBytes = static_cast<size_t>(WAVES) * kI8pXBytes;
    __shared__ __align__(16) unsigned char lds_raw[kRedBytes > kXchBytes ? kRedBytes : kXchBytes];
    float (*const red)[NB * MB][4][kWave] = reinterpret_cast<float (*)[NB * MB][4][kWave]>(lds_raw);
    unsigned char (*const xch_all)[kI8pXBytes] = reinterpret_cast<unsigned char (*)[kI8pXBytes]>(lds_raw);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int steps = K / 128;
    const int n0 = blockIdx.x * (16 * NB);
    const uint4* w_base[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int n = n0 + 16 * b + i;
        w_base[b] = reinterpret_cast<const uint4*>(w + static_cast<size_t>(n < N ? n : N - 1) * K) + q * 2;  // rows past N: a valid row, result dropped
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
    unsigned char* const xch_put = xch_all[wave] + (lane >> 4) * kI8pXPitch + (lane & 15) * 16;  // + 4 j' rows
    const unsigned char* const xch_get = xch_all[wave] + i * kI8pXPitch + q * 64;                 // + 16 c

    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 bias = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
    uint32_t magic;  // exponent bytes, kept in a VGPR behind an opaque move
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(0x64646464u));

    struct Step {
        uint4 w[NB][2];
        uint4 xv[MB][4];
    };
    auto load = [&](int s, Step& st) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            st.w[b][0] = nt_load(w_base[b] + s * 8);
            st.w[b][1] = nt_load(w_base[b] + s * 8 + 1);
        }
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) st.xv[r][c] = x_base[4 * r + c][s * 16];  // as loaded: rows 16 r + 4 c .. + 3
    };
    float4_t d[NB][MB][2] = {};  // two accumulators per output block taking turns
    auto compute = [&](const Step& st) {
        // each block of 16 rows into the exchange area and this lane's four pieces out of it (LDS keeps a wavefront's
        // accesses in order: the reads of the block before are served before these writes)
        uint4 xb[MB][4];
#pragma unroll
        for (int r = 0; r < MB; ++r) {
#pragma unroll
            for (int c = 0; c < 4; ++c) *reinterpret_cast<uint4*>(xch_put + c * 4 * kI8pXPitch) = st.xv[r][c];
#pragma unroll
            for (int c = 0; c < 4; ++c) xb[r][c] = *reinterpret_cast<const uint4*>(xch_get + c * 16);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {  // MFMA u (16x16x32): k = 8u .. 8u+7 of the lane's 32
            word4_t bv[MB];
#pragma unroll
            for (int r = 0; r < MB; ++r) bv[r] = word4_t{xb[r][u].x, xb[r][u].y, xb[r][u].z, xb[r][u].w};
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                uint32_t a[4];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t word = dword_at(st.w[b][u >> 1], (2 * u + h) & 3);
                    if constexpr (DT == TPQ_DTYPE_F16) {
                        const uint32_t t = word ^ 0x80808080u;
                        const uint32_t lo = __builtin_amdgcn_perm(magic, t, 0x04010400u);  // (1152 + b0, 1152 + b1)
                        const uint32_t hi = __builtin_amdgcn_perm(magic, t, 0x04030402u);  // (1152 + b2, 1152 + b3)
                        a[2 * h] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, lo) - bias);
                        a[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, hi) - bias);
                    } else {
                        // bf16 is the upper half of a float and an int8 has eight significant bits: convert each
                        // byte (sign-extending byte select) and keep the upper halves, exact
                        uint32_t f[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) f[e] = __builtin_bit_cast(uint32_t, static_cast<float>(static_cast<int8_t>(word >> (8 * e))));
                        a[2 * h] = __builtin_amdgcn_perm(f[1], f[0], 0x07060302u);      // (bf16 b0, bf16 b1)
                        a[2 * h + 1] = __builtin_amdgcn_perm(f[3], f[2], 0x07060302u);  // (bf16 b2, bf16 b3)
                    }
                }
                const word4_t av = {a[0], a[1], a[2], a[3]};
#pragma unroll
                for (int r = 0; r < MB; ++r) {
                    float4_t& acc = d[b][r][u & 1];
                    if constexpr (DT == TPQ_DTYPE_F16)
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, av), __builtin_bit_cast(half8_t, bv[r]), acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, av), __builtin_bit_cast(bf8_t, bv[r]), acc, 0, 0, 0);
                }
            }
        }
    };

    // this wavefront's steps: wave, wave + W, ...; kI8Ring of them in flight
    Step ring[kI8Ring] = {};
#pragma unroll
    for (int r = 0; r < kI8Ring; ++r)
        if (wave + r * WAVES < steps) load(wave + r * WAVES, ring[r]);
    for (int base = wave; base < steps; base += kI8Ring * WAVES) {
#pragma unroll
        for (int r = 0; r < kI8Ring; ++r) {
            const int s = base + r * WAVES;
            if (s < steps) {
                compute(ring[r]);
                if (s + kI8Ring * WAVES < steps) load(s + kI8Ring * WAVES, ring[r]);
            }
        }
    }

    float scale_n[NB][4];  // the finishing wavefront's channel scales, asked for ahead of the exchange
    if (wave == 0) {
        const auto sp = pinned_global(scale);
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int n = n0 + 16 * b + 4 * q + v;
                scale_n[b][v] = sp[n < N ? n : N - 1];
            }
    }
    __syncthreads();  // every wavefront is done with its exchange area
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][b * MB + r][v][lane] = d[b][r][0][v] + d[b][r][1][v];
    __syncthreads();
    if (wave == 0) {  // lane (m, q): rows 16 r + m, channels n0 + 16 b + 4 q + v
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int r = 0; r < MB; ++r)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float sum = 0.0f;
#pragma unroll
                    for (int ww = 0; ww < WAVES; ++ww) sum += red[ww][b * MB + r][v][lane];
                    const int n = n0 + 16 * b + 4 * q + v;
                    if (row_live[r] && n < N) y[static_cast<size_t>(16 * r + i) * N + n] = Elem<DT>::store(__fmul_rn(sum, scale_n[b][v]));
                }
    }
}

// One or two activation rows (fp16 / bf16, K % 16 == 0, K <= 65536; two rows: K <= 32768, at most eight wavefronts):
// the weight rows are contiguous, so a wavefront reads a
// row's bytes directly: lane l owns the 16 k of chunk 64 t + l of its pass (a pass = four such turns = 4096 k), one
// 16-byte load per turn and channel, 1 KB contiguous per wavefront and load, and the 32 bytes of activations that go
// with them, shared by the wavefront's four channels.  Every load of a wavefront is issued before the first use, so
// the whole weight is in flight within the first microsecond, as in the int4 kernel for one row.  A workgroup of
// 4, 8 or 16 wavefronts = channel groups x passes (the fewer, the more workgroups: small weights need them to fill the chip); the lanes' sums meet by a butterfly, the passes' through LDS.
// fp16: bytes -> fp16 pairs as in the kernel above, v_dot2_f32_f16; bf16: both operands widened to fp32, fma.
constexpr int kRowChannels = 4, kRowTurns = 4;

template <int DT, int kRowWaves, int ROWS>
__global__ __launch_bounds__(kRowWaves * kWave) void int8pack_row_kernel(const uint16_t* __restrict__ x, const int8_t* __restrict__ w,
                                                                        const float* __restrict__ scale, uint16_t* __restrict__ y,
                                                                        int N, int K, int passes, int groups) {
    __shared__ float red[kRowWaves][kRowChannels * ROWS];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = wave / passes, pass = wave - g * passes;
    const int n0 = (blockIdx.x * groups + g) * kRowChannels;
    const bool active = g < groups && n0 < N;
    // thread = (group, channel, row) finishes one output; its channel scale is asked for ahead of the weights
    const int tid = threadIdx.x;
    const int out_group = tid / (kRowChannels * ROWS), out_rem = tid - out_group * (kRowChannels * ROWS);
    const int out_c = out_rem / ROWS, out_r = out_rem - out_c * ROWS;
    const int out_n = (blockIdx.x * groups + out_group) * kRowChannels + out_c;
    const bool finishes = tid < groups * kRowChannels * ROWS && out_n < N;
    float scale_n = 0.0f;
    if (finishes) scale_n = pinned_global(scale)[out_n];
    float acc[kRowChannels][ROWS];
#pragma unroll
    for (int c = 0; c < kRowChannels; ++c)
#pragma unroll
        for (int r = 0; r < ROWS; ++r) acc[c][r] = 0.0f;
    if (active) {
        const int chunks = K >> 4;
        uint4 wv[kRowChannels][kRowTurns];
        uint4 xv[ROWS][kRowTurns][2];
        bool live[kRowTurns];
#pragma unroll
        for (int t = 0; t < kRowTurns; ++t) {
            const int chunk = (pass * kRowTurns + t) * kWave + lane;
            live[t] = chunk < chunks;
            const int cl = live[t] ? chunk : chunks - 1;  // past the end: a valid chunk, multiplied by zeros
#pragma unroll
            for (int c = 0; c < kRowChannels; ++c) {
                const int n = n0 + c < N ? n0 + c : N - 1;
                wv[c][t] = nt_load(reinterpret_cast<const uint4*>(w + static_cast<size_t>(n) * K) + cl);
            }
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const uint4* xp = reinterpret_cast<const uint4*>(x + static_cast<size_t>(r) * K) + 2 * cl;
                xv[r][t][0] = live[t] ? xp[0] : make_uint4(0, 0, 0, 0);
                xv[r][t][1] = live[t] ? xp[1] : make_uint4(0, 0, 0, 0);
            }
        }
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 bias = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
        uint32_t magic;  // exponent bytes, kept in a VGPR behind an opaque move
        asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(0x64646464u));
#pragma unroll
        for (int t = 0; t < kRowTurns; ++t) {
#pragma unroll
            for (int c = 0; c < kRowChannels; ++c) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {  // dword j: k = 4 j .. 4 j + 3 of the chunk
                    const uint32_t word = dword_at(wv[c][t], j);
                    if constexpr (DT == TPQ_DTYPE_F16) {
                        const uint32_t u = word ^ 0x80808080u;
                        const h2 lo = __builtin_bit_cast(h2, __builtin_amdgcn_perm(magic, u, 0x04010400u)) - bias;  // (b0, b1)
                        const h2 hi = __builtin_bit_cast(h2, __builtin_amdgcn_perm(magic, u, 0x04030402u)) - bias;  // (b2, b3)
#pragma unroll
                        for (int r = 0; r < ROWS; ++r) {
                            const uint4& xq = xv[r][t][j >> 1];
                            const uint32_t x0 = (j & 1) ? xq.z : xq.x, x1 = (j & 1) ? xq.w : xq.y;
                            acc[c][r] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, x0), lo, acc[c][r], false);
                            acc[c][r] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, x1), hi, acc[c][r], false);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float wf = static_cast<float>(static_cast<int8_t>(word >> (8 * e)));
#pragma unroll
                            for (int r = 0; r < ROWS; ++r) {
                                const uint4& xq = xv[r][t][j >> 1];
                                const uint32_t xp2 = (j & 1) ? ((e >> 1) ? xq.w : xq.z) : ((e >> 1) ? xq.y : xq.x);
                                const float xf = __builtin_bit_cast(float, (e & 1) ? (xp2 & 0xFFFF0000u) : (xp2 << 16));
                                acc[c][r] = __builtin_fmaf(xf, wf, acc[c][r]);
                            }
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < kRowChannels; ++c)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) acc[c][r] = wave_sum(acc[c][r]);
    }
    if (lane == 0) {
#pragma unroll
        for (int c = 0; c < kRowChannels; ++c)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) red[wave][c * ROWS + r] = acc[c][r];
    }
    __syncthreads();
    if (finishes) {  // the passes in order
        float sum = 0.0f;
        for (int ps = 0; ps < passes; ++ps) sum += red[out_group * passes + ps][out_rem];
        y[static_cast<size_t>(out_r) * N + out_n] = Elem<DT>::store(__fmul_rn(sum, scale_n));
    }
}

// Any floating activation dtype, K % 8 == 0, 16-byte aligned rows: a wavefront owns four consecutive output
// channels and a slab of up to four activation rows; a lane takes eight consecutive k per turn (8 bytes of
// each weight row, 16 or 32 bytes of each activation row), fp32 fma, one wavefront reduction at the end.
constexpr int kVecChannels = 4, kVecRows = 4;

template <int DT>
__global__ __launch_bounds__(256) void int8pack_vector_kernel(
    const typename Elem<DT>::storage* __restrict__ x, const int8_t* __restrict__ w, const float* __restrict__ scale,
    typename Elem<DT>::storage* __restrict__ y, int64_t M, int64_t N, int64_t K) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int64_t n0 = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * kVecChannels, m0 = static_cast<int64_t>(blockIdx.y) * kVecRows;
    if (n0 >= N) return;
    const int rows = static_cast<int>(M - m0 < kVecRows ? M - m0 : kVecRows);
    float acc[kVecChannels][kVecRows];
#pragma unroll
    for (int c = 0; c < kVecChannels; ++c)
#pragma unroll
        for (int r = 0; r < kVecRows; ++r) acc[c][r] = 0.0f;
    for (int64_t k = static_cast<int64_t>(lane) * 8; k < K; k += kWave * 8) {
        float xv[kVecRows][8];
#pragma unroll
        for (int r = 0; r < kVecRows; ++r)
            if (r < rows) load_eight<DT>(x + (m0 + r) * K + k, xv[r]);
#pragma unroll
        for (int c = 0; c < kVecChannels; ++c) {
            const int64_t n = n0 + c < N ? n0 + c : N - 1;  // channels past N: a valid row, result dropped
            const uint2 raw = nt_load(reinterpret_cast<const uint2*>(w + n * K + k));
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t word = e < 4 ? raw.x : raw.y;
                const float wv = static_cast<float>(static_cast<int8_t>(word >> (8 * (e & 3))));
#pragma unroll
                for (int r = 0; r < kVecRows; ++r)
                    if (r < rows) acc[c][r] = __builtin_fmaf(wv, xv[r][e], acc[c][r]);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < kVecChannels; ++c)
#pragma unroll
        for (int r = 0; r < kVecRows; ++r) {
            const float total = wave_sum(acc[c][r]);
            if (lane == 0 && r < rows && n0 + c < N) y[(m0 + r) * N + n0 + c] = Elem<DT>::store(__fmul_rn(total, scale[n0 + c]));
        }
}

// One workgroup per output channel n and slab of up to 8 activation rows.
template <int DT>
__global__ __launch_bounds__(256) void int8pack_generic_kernel(
    const typename Elem<DT>::storage* __restrict__ x, const int8_t* __restrict__ w, const float* __restrict__ scale,
    typename Elem<DT>::storage* __restrict__ y, int64_t M, int64_t N, int64_t K) {
    __shared__ float red[8][256 / kWave];
    const int64_t n = blockIdx.x, m0 = static_cast<int64_t>(blockIdx.y) * 8;
    const int rows = static_cast<int>(M - m0 < 8 ? M - m0 : 8);
    const int8_t* wr = w + n * K;
    float acc[8];
#pragma unroll
    for (int b = 0; b < 8; ++b) acc[b] = 0.0f;
    for (int64_t k = threadIdx.x; k < K; k += 256) {
        const float wv = static_cast<float>(wr[k]);
#pragma unroll
        for (int b = 0; b < 8; ++b)
            if (b < rows) acc[b] = __builtin_fmaf(wv, Elem<DT>::load(x[(m0 + b) * K + k]), acc[b]);
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        float v = acc[b];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
        if (lane == 0) red[b][wave] = v;
    }
    __syncthreads();
    if (threadIdx.x < rows) {
        const int b = threadIdx.x;
        const float total = (red[b][0] + red[b][1]) + (red[b][2] + red[b][3]);
        y[(m0 + b) * N + n] = Elem<DT>::store(__fmul_rn(total, scale[n]));
    }
}

template <int DT>
int launch_generic(const void* x, const int8_t* w, const float* scale, void* y, int64_t M, int64_t N, int64_t K, hipStream_t s) {
    using S = typename Elem<DT>::storage;
    if (K % 8 == 0 && aligned(x, 32) && aligned(w, 8)) {
        const int64_t gx = (N + 4 * kVecChannels - 1) / (4 * kVecChannels), gy = (M + kVecRows - 1) / kVecRows;
        TPQ_REQUIRE(gx <= 0x7FFFFFFF && gy <= 65535, TPQ_ERR_INVALID_VALUE, "_weight_int8pack_mm(): shape too large");
        int8pack_vector_kernel<DT><<<dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)), 256, 0, s>>>(
            static_cast<const S*>(x), w, scale, static_cast<S*>(y), M, N, K);
        return check_launch("_weight_int8pack_mm (vector)");
    }
    const int64_t slabs = (M + 7) / 8;
    TPQ_REQUIRE(N <= 0x7FFFFFFF && slabs <= 65535, TPQ_ERR_INVALID_VALUE, "_weight_int8pack_mm(): shape too large");
    int8pack_generic_kernel<DT><<<dim3(static_cast<unsigned>(N), static_cast<unsigned>(slabs)), 256, 0, s>>>(
        static_cast<const S*>(x), w, scale, static_cast<S*>(y), M, N, K);
    return check_launch("_weight_int8pack_mm (generic)");
}

// Dense [N, K] weight of `DT`: T(float(w) * scale[n]), one rounding; thread = 16 consecutive k of a row
// (K % 16 == 0) or, for other K, one element.
template <int DT>
__global__ __launch_bounds__(256) void int8pack_dequantize_kernel(const int8_t* __restrict__ w, const float* __restrict__ scale,
                                                                  typename Elem<DT>::storage* __restrict__ out, int64_t N, int64_t K,
                                                                  int vectors) {
    using S = typename Elem<DT>::storage;
    if (vectors) {
        const int64_t chunks = N * K / 16;
        for (int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; c < chunks; c += static_cast<int64_t>(gridDim.x) * blockDim.x) {
            const float sc = scale[(c * 16) / K];
            const uint4 raw = nt_load(reinterpret_cast<const uint4*>(w) + c);
            const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
            __attribute__((aligned(16))) S o[16];
#pragma unroll
            for (int e = 0; e < 16; ++e)
                o[e] = Elem<DT>::store(__fmul_rn(static_cast<float>(static_cast<int8_t>(words[e >> 2] >> (8 * (e & 3)))), sc));
            uint4* dst = reinterpret_cast<uint4*>(out + c * 16);
#pragma unroll
            for (int e = 0; e < static_cast<int>(16 * sizeof(S) / 16); ++e) dst[e] = reinterpret_cast<const uint4*>(o)[e];
        }
    } else {
        for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < N * K; i += static_cast<int64_t>(gridDim.x) * blockDim.x)
            out[i] = Elem<DT>::store(__fmul_rn(static_cast<float>(w[i]), scale[i / K]));
    }
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int tpq_int8pack_dequantize(const int8_t* w, const float* scales, int64_t N, int64_t K, int dtype, void* out, void* stream) {
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F32 || dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16, TPQ_ERR_INVALID_TYPE,
                "int8pack dequantize: the dense weight must be floating point");
    TPQ_REQUIRE(N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "int8pack dequantize: negative shape");
    if (N == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(w && scales && out, TPQ_ERR_INVALID_VALUE, "int8pack dequantize: null pointer");
    const int vectors = K % 16 == 0 && aligned(w, 16) && aligned(out, 16);
    const int64_t items = vectors ? N * K / 16 : N * K;
    const int64_t blocks = (items + 255) / 256;
    const unsigned grid = static_cast<unsigned>(blocks > (1 << 20) ? (1 << 20) : blocks);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case TPQ_DTYPE_F32: int8pack_dequantize_kernel<TPQ_DTYPE_F32><<<grid, 256, 0, s>>>(w, scales, static_cast<float*>(out), N, K, vectors); break;
        case TPQ_DTYPE_F16: int8pack_dequantize_kernel<TPQ_DTYPE_F16><<<grid, 256, 0, s>>>(w, scales, static_cast<uint16_t*>(out), N, K, vectors); break;
        default: int8pack_dequantize_kernel<TPQ_DTYPE_BF16><<<grid, 256, 0, s>>>(w, scales, static_cast<uint16_t*>(out), N, K, vectors); break;
    }
    return check_launch("tpq_int8pack_dequantize");
}

TPQ_EXPORT int tpq_weight_int8pack_mm(const void* x, int dtype, int64_t M, int64_t K, const int8_t* w,
                                      const float* scales, int64_t N, void* out, void* stream) {
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F32 || dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16, TPQ_ERR_INVALID_TYPE,
                "_weight_int8pack_mm(): activations must be floating point");
    TPQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "_weight_int8pack_mm(): negative shape");
    if (M == 0 || N == 0 || K == 0) return TPQ_OK;  // the reference returns an uninitialised [B, N] here
    TPQ_REQUIRE(x && w && scales && out, TPQ_ERR_INVALID_VALUE, "_weight_int8pack_mm(): null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    // One row: the row kernel, at every shape (measured against the matrix-core kernel below, us: 4096 x 4096 5.8 / 6.4,
    // 11008 -> 4096 10.8 / 14.3, 4096 -> 11008 10.6 / 12.9, 8192 x 8192 13.8 / 18.5, 8192 -> 28672 40.1 / 53.7, 28672 -> 8192
    // 39.7 / 54.4, 2560 -> 6912 6.2 / 7.8).  Workgroup size by the size of the weight: small weights need many
    // workgroups to fill the chip (4096 x 4096: 5.8 us with 4 wavefronts, 8.9 with 16), the largest stream best with 8
    // (8192 -> 28672: 40.1 us = 5.9 TB/s; 42.0 with 4, 45.1 with 16).  TPQ_INT8PACK_ROW=0 / 1 pins the kernel and
    // TPQ_INT8PACK_ROW_WAVES the workgroup size for comparison runs.
    static const int forced_row = [] { const char* e = tuning_env("TPQ_INT8PACK_ROW"); return e ? std::atoi(e) : -1; }();
    static const int forced_row_waves = [] { const char* e = tuning_env("TPQ_INT8PACK_ROW_WAVES"); return e ? std::atoi(e) : 0; }();
    if (M <= 2 && dtype != TPQ_DTYPE_F32 && K % 16 == 0 && K <= (M == 1 ? 65536 : 32768) && N <= 0x7FFFFFF0 && aligned(x, 16) && aligned(w, 16) && forced_row != 0) {
        const int passes = static_cast<int>((K + 4095) / 4096);
        int waves = N * K >= (int64_t{1} << 27) ? 8 : N * K >= (int64_t{1} << 26) ? 16 : 4;
        if (forced_row_waves == 4 || forced_row_waves == 8 || forced_row_waves == 16) waves = forced_row_waves;
        if (M == 2 && waves == 16) waves = 8;  // two rows: 64 more registers of activations per lane
        while (waves < passes) waves *= 2;  // a workgroup holds all passes of its channels
        const int groups = waves / passes;
        const dim3 grid(static_cast<unsigned>((N + groups * kRowChannels - 1) / (groups * kRowChannels)));
        const auto* xp = static_cast<const uint16_t*>(x);
        auto* yp = static_cast<uint16_t*>(out);
#define TPQ_I8ROW_R(DTV, WV, RV) int8pack_row_kernel<DTV, WV, RV><<<grid, WV * kWave, 0, s>>>(xp, w, scales, yp, (int)N, (int)K, passes, groups)
#define TPQ_I8ROW(DTV, WV) do { if (M == 1) TPQ_I8ROW_R(DTV, WV, 1); else if (WV <= 8) TPQ_I8ROW_R(DTV, WV, (WV <= 8 ? 2 : 1)); } while (0)
        if (dtype == TPQ_DTYPE_F16) { if (waves == 4) TPQ_I8ROW(TPQ_DTYPE_F16, 4); else if (waves == 8) TPQ_I8ROW(TPQ_DTYPE_F16, 8); else TPQ_I8ROW(TPQ_DTYPE_F16, 16); }
        else { if (waves == 4) TPQ_I8ROW(TPQ_DTYPE_BF16, 4); else if (waves == 8) TPQ_I8ROW(TPQ_DTYPE_BF16, 8); else TPQ_I8ROW(TPQ_DTYPE_BF16, 16); }
#undef TPQ_I8ROW
#undef TPQ_I8ROW_R
        return check_launch("_weight_int8pack_mm (row)");
    }
    if (dtype != TPQ_DTYPE_F32 && K % 128 == 0 && K <= 0x7FFFFF80 && N <= 0x7FFFFFF0 && aligned(x, 16) && aligned(w, 16)) {
        static const int forced_nb = [] { const char* e = tuning_env("TPQ_INT8PACK_NB"); return e ? std::atoi(e) : 0; }();
        static const int forced_waves = [] { const char* e = tuning_env("TPQ_INT8PACK_WAVES"); return e ? std::atoi(e) : 0; }();
        static const int forced_mb = [] { const char* e = tuning_env("TPQ_INT8PACK_MB"); return e ? std::atoi(e) : 0; }();
        for (int64_t m0 = 0; m0 < M;) {
            const int left = static_cast<int>(M - m0 < 32 ? M - m0 : 32);
            if (N <= 0x7FFFFFF0 && K <= 0x7FFFFF80) {  // the all-in-flight form, where it is built (17..32 rows: two blocks of 16)
                int rc = TPQ_OK;
                if (flight_launch_int8pack(dtype, static_cast<const uint16_t*>(x) + m0 * K, left, w, scales, static_cast<uint16_t*>(out) + m0 * N,
                                           static_cast<int>(N), static_cast<int>(K), s, &rc)) {
                    if (rc != TPQ_OK) return rc;
                    m0 += left;
                    continue;
                }
            }
            const int mb = forced_mb ? forced_mb : (left > 16 ? 2 : 1);
            const int rows = left < 16 * mb ? left : 16 * mb;
            // Workgroup shape from a sweep over model shapes (K, N = 1024..28672; 1, 8, 16 rows): 16 channels x 8
            // wavefronts (4096 x 4096, one row: 6.4 us; 2 wavefronts 9.5); 32 channels for N = 4097 .. 10239, where 16-channel
            // workgroups would outnumber the compute units by less than two (13824 -> 5120, 8 rows: 28.6 us against 34.6;
            // 4096 -> 6144, 16 rows: 12.6 against 14.8), and from 8 rows on at N >= 16384 (28672 -> 8192, 16 rows: 72 us against 88).
            const bool wide = (N > 4096 && N < 10240) || (N >= 16384 && rows >= 8);
            const int nb = forced_nb ? forced_nb : (wide ? 2 : 1);
            const int waves = forced_waves ? forced_waves : (N >= 16384 && !wide ? 4 : 8);
            const dim3 grid(static_cast<unsigned>((N + 16 * nb - 1) / (16 * nb)));
            const auto* xs = static_cast<const uint16_t*>(x) + m0 * K;
            auto* ys = static_cast<uint16_t*>(out) + m0 * N;
            const int n = static_cast<int>(N), k = static_cast<int>(K);
#define TPQ_I8P(DTV, NBV, MBV, WV) int8pack_mfma_kernel<DTV, NBV, MBV, WV><<<grid, WV * kWave, 0, s>>>(xs, w, scales, ys, rows, n, k)
#define TPQ_I8P_DT(NBV, MBV, WV) do { if (dtype == TPQ_DTYPE_F16) TPQ_I8P(TPQ_DTYPE_F16, NBV, MBV, WV); else TPQ_I8P(TPQ_DTYPE_BF16, NBV, MBV, WV); } while (0)
            if (mb == 2) {
                if (nb == 2) { if (waves == 4) TPQ_I8P_DT(2, 2, 4); else TPQ_I8P_DT(2, 2, 8); }
                else { if (waves == 4) TPQ_I8P_DT(1, 2, 4); else TPQ_I8P_DT(1, 2, 8); }
            } else if (nb == 2) { if (waves == 8) TPQ_I8P_DT(2, 1, 8); else if (waves == 4) TPQ_I8P_DT(2, 1, 4); else TPQ_I8P_DT(2, 1, 2); }
            else { if (waves == 8) TPQ_I8P_DT(1, 1, 8); else if (waves == 4) TPQ_I8P_DT(1, 1, 4); else TPQ_I8P_DT(1, 1, 2); }
#undef TPQ_I8P_DT
#undef TPQ_I8P
            m0 += rows;
        }
        return check_launch("_weight_int8pack_mm (mfma)");
    }
    switch (dtype) {
        case TPQ_DTYPE_F32: return launch_generic<TPQ_DTYPE_F32>(x, w, scales, out, M, N, K, s);
        case TPQ_DTYPE_F16: return launch_generic<TPQ_DTYPE_F16>(x, w, scales, out, M, N, K, s);
        default: return launch_generic<TPQ_DTYPE_BF16>(x, w, scales, out, M, N, K, s);
    }
}
