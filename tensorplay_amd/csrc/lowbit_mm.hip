// Weight-only matmul for the packed n-bit weights (1 <= bits <= 8) of the reference's int2 / intx /
// binary weight-only modules:
//   out[m, n] = sum_k x[m, k] * (code[n, k] - zero[g, n]) * scale[g, n]  (+ bias[n]),  g = k / group
// packed: uint8 [N, ceil(K / per_byte)], per_byte = 8 / bits codes per byte, code i of a byte in bits
// 8 - (i + 1) * bits .. (first code in the most significant bits: pack_intx / pack_int2,
// tensorplay/ao/quantization/intx_weight_only.py:35-59, int2_weight_only.py:63-88) or, for the 1-bit
// sign weights, in bit i (pack_binary, binary.py:50-71).  scales_and_zeros: f32 [K / group][N][2], the
// buffer the modules keep (intx_weight_only.py:167-170).  The reference unpacks with tensor ops,
// dequantizes to a dense float weight and calls a float GEMM (_intx_mm, intx_weight_only.py:127-133).
//
// Decode kernel (fp16 / bf16 activations, 1..16 rows): v_mfma_f32_16x16x32 with the weights as A (fp16 below;
// bf16 the same with seven mantissa bits, see Fields).  Lane
// (i, q) owns weight row n0 + i and, per step, 32 consecutive codes of it (16 when a code has a byte
// to itself): 4 to 16 bytes, one load.  A code becomes an fp16 number without leaving its bits: the
// byte is copied into both halves of a dword (v_perm_b32), a mask keeps one field per half and an
// exponent is or-ed in, chosen so that the field's position in the mantissa has weight one: a field at
// bit p under exponent 2^(10-p) reads 2^(10-p) + code.  Two neighbouring codes per dword, so the B
// operand is simply the activations as they lie in memory.  The offsets 2^(10-p) leave through one
// more MFMA per eight k whose A is constant (row 0: the offsets, row 1: ones -> sum of x), and a step
// stays inside one quantization group:  y += scale * ((D - offsets) - zero * sum x).
//
// Everything else (fp32 / bf16 activations, other group sizes) takes the vector kernel below (wavefront = four
// channels, eight k per lane and turn), and K or group sizes that are not multiples of 8 a plain one: one
// workgroup per output channel and slab of up to 8 rows; both form the dequantized weight in fp32 exactly as the
// reference does and accumulate with fp32 fma.
#include <cstdlib>

#include "int4_lane.h"

namespace tpq {
namespace {

typedef uint32_t word4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

// dword r of a 16-byte vector; r is a constant once the loops around the call are unrolled
__device__ __forceinline__ uint32_t dword_at(const uint4& q, int r) { return r == 0 ? q.x : r == 1 ? q.y : r == 2 ? q.z : q.w; }

template <int BITS, bool LSB>
struct Fields {
    static constexpr int kPerByte = 8 / BITS;
    static constexpr int kCodes = kPerByte >= 2 ? 32 : 16;  // per lane and step
    static constexpr int kBytes = kCodes / kPerByte;        // 4, 8 or 16
    static constexpr int kStepK = 4 * kCodes;
    static constexpr uint32_t kField = (1u << BITS) - 1u;
    // bit position of code i of a byte
    static constexpr int pos(int i) { return LSB ? i * BITS : 8 - (i + 1) * BITS; }
    // fp16 bits of 2^(10 - p): a field at bit p of the mantissa then counts in units of one
    static constexpr uint32_t base_bits(int p) { return static_cast<uint32_t>(25 - p) << 10; }
    // pair t = codes 2t, 2t + 1 of the lane's bytes: which byte goes to which half, masks, exponents
    static constexpr int byte_lo(int t) { return (2 * t) / kPerByte; }
    static constexpr int byte_hi(int t) { return (2 * t + 1) / kPerByte; }
    static constexpr int pos_lo(int t) { return pos((2 * t) % kPerByte); }
    static constexpr int pos_hi(int t) { return pos((2 * t + 1) % kPerByte); }
    static constexpr uint32_t select(int t) { return 0x0C000C00u | (byte_lo(t) & 3) | ((byte_hi(t) & 3) << 16); }
    static constexpr uint32_t mask(int t) { return (kField << pos_lo(t)) | (kField << (pos_hi(t) + 16)); }
    static constexpr uint32_t magic(int t) { return base_bits(pos_lo(t)) | (base_bits(pos_hi(t)) << 16); }
    static constexpr int kMagics = kPerByte >= 2 ? kPerByte / 2 : 1;  // magic(t) repeats with this period
    // bfloat16 (BITS < 8): seven mantissa bits, so the top field of a byte reaches into the exponent.  It is taken from
    // the word shifted right by one (its byte then holds the field one bit lower; the bit that comes in from the next
    // byte is masked away): v_perm_b32 picks each half's byte from the word or from the shifted word.
    static constexpr bool top(int p) { return p + BITS > 7; }
    static constexpr int pos_bf(int p) { return top(p) ? p - 1 : p; }
    static constexpr uint32_t base_bits_bf(int p) { return static_cast<uint32_t>(127 + 7 - p) << 7; }  // bf16 bits of 2^(7 - p)
    static constexpr uint32_t select_bf(int t) {
        return 0x0C000C00u | ((byte_lo(t) & 3) + (top(pos_lo(t)) ? 4 : 0)) | (((byte_hi(t) & 3) + (top(pos_hi(t)) ? 4 : 0)) << 16);
    }
    static constexpr uint32_t mask_bf(int t) { return (kField << pos_bf(pos_lo(t))) | (kField << (pos_bf(pos_hi(t)) + 16)); }
    static constexpr uint32_t magic_bf(int t) { return base_bits_bf(pos_bf(pos_lo(t))) | (base_bits_bf(pos_bf(pos_hi(t))) << 16); }
};

typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));

// 8-bit codes are signed in the reference: unpack_intx ends in codes.to(int8) and _dequantize_intx converts that int8
// to float (tensorplay/ao/quantization/intx_weight_only.py:62-80, 110-124), so a byte of 128 or more counts as
// byte - 256.  The matrix-core and row kernels keep their unsigned field arithmetic: byte ^ 0x80 = value + 128, so
// the packed words are flipped after the load and 128 is added to the zero point.
constexpr uint32_t kSignFlip = 0x80808080u;

// x: [M][K] fp16 or bf16; packed: [N][K / per_byte]; sz: [K / group][N][2] fp32; steps = K / kStepK; a group
// is kStepK << group_shift k.  N % 4 == 0.
// bf16 has seven mantissa bits: the same exponent trick with the top field of every byte taken from the word shifted
// right by one bit (Fields::select_bf); only at 8 bits, where a byte does not fit, a code is cut out of its dword,
// converted to float (exact) and the upper halves of two floats are packed, with no offsets to take out (the
// constant-A MFMA then only sums x).
//
// The activations of a step are kStepK * 2 bytes of every row.  Asked for in the MFMA's order (lane (m, q): its 16-byte
// pieces of row m) every load touches two or three lines of every row, and the vector memory path charges a load by the
// lines it touches: at 8 rows the activations cost it four times what the packed weights do, and the time grew by half a
// microsecond per row.  So a wavefront reads them as they lie (a load = 64 consecutive 16-byte pieces = 4 or 8 whole
// rows of the step, XL loads for up to 16 rows) and passes them to the MFMA's lanes through a wave-private LDS area
// whose rows are 16 bytes longer than a step, so that the sixteen rows of a 16-byte read spread over the banks.
// Columns m >= M hold whatever is there; their sums are dropped.  Measured, 4096 -> 11008, 1 / 2 / 4 bits (us, with the
// loads in MFMA order -> as they lie): 2 rows 10.0 / 10.4 / 10.7 -> 9.2 / 9.0 / 10.4, 4 rows 11.1 / 11.4 / 11.6 ->
// 9.4 / 9.1 / 11.6, 8 rows 13.2 / 13.4 / 13.6 -> 12.3 / 11.0 / 11.5, 16 rows 17.1 / 17.7 / 17.7 -> 12.8 / 12.4 / 13.4.
template <int BITS, bool LSB>
constexpr int lowbit_x_pitch() { return Fields<BITS, LSB>::kStepK * 2 + 16; }

// NB blocks of 16 channels per workgroup share the activations of a step: every workgroup pulls all activation rows
// through its compute unit, so with one block the activations outweigh a narrow packed weight many times over.
// 4096 -> 11008 with three blocks against one (us, 1 / 2 / 4 bits): 2 rows 9.2 / 9.0 / 10.4 -> 8.2 / 8.6 / 9.3, 8 rows
// 12.3 / 11.0 / 11.5 -> 9.9 / 10.5 / 11.1, 16 rows 12.8 / 12.4 / 13.4 -> 10.5 / 10.9 / 11.6.
// bfloat16 with the fields expanded in place instead of converted one by one (2 / 8 rows, us): 1 bit 9.7 / 10.3 -> 8.4 / 9.1,
// 2 bits 10.0 / 10.7 -> 9.3 / 10.0, 4 bits 10.5 / 10.9 -> 9.5 / 10.5.
template <int DT, int BITS, bool LSB, int WAVES, int XL, int NB>
__global__ __launch_bounds__(WAVES * kWave) void lowbit_mfma_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ packed, const float* __restrict__ sz,
    const float* __restrict__ bias, uint16_t* __restrict__ y, int M, int N, int K, int group_shift) {
    using F = Fields<BITS, LSB>;
    constexpr int kPiecesPerRow = F::kStepK / 8;           // 16-byte pieces of a row and step: 16, or 8 at one code per byte
    constexpr int kRowsPerLoad = kWave / kPiecesPerRow;    // 4 or 8
    constexpr int kPitch = lowbit_x_pitch<BITS, LSB>();
    static_assert(XL * kRowsPerLoad <= 16, "at most 16 rows per launch");
    constexpr bool kFieldsInPlace = DT == TPQ_DTYPE_F16 || BITS < 8;  // codes become 16-bit floats without leaving their bits
    __shared__ float red[WAVES][NB * 4][kWave];
    extern __shared__ __align__(16) unsigned char lowbit_xch[];  // [WAVES][16 rows][kPitch]
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int steps = K / F::kStepK;
    const int n0 = blockIdx.x * (16 * NB);
    const uint8_t* w_base[NB];
    const float* sz_base[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int n_row = n0 + 16 * b + i < N ? n0 + 16 * b + i : N - 1;  // rows past N: a valid row, result dropped
        w_base[b] = packed + static_cast<size_t>(n_row) * (K / F::kPerByte) + q * F::kBytes;
        int n4 = n0 + 16 * b + 4 * q;  // this lane's four output channels of the block
        n4 = n4 + 4 <= N ? n4 : N - 4;
        sz_base[b] = sz + static_cast<size_t>(n4) * 2;
    }
    const bool row_live = i < M;
    // load j of a step: row kRowsPerLoad j + lane / kPiecesPerRow, piece lane % kPiecesPerRow (rows past M: row 0, dropped)
    const uint4* x_base[XL];
#pragma unroll
    for (int j = 0; j < XL; ++j) {
        const int row = kRowsPerLoad * j + lane / kPiecesPerRow;
        x_base[j] = reinterpret_cast<const uint4*>(x + static_cast<size_t>(row < M ? row : 0) * K) + lane % kPiecesPerRow;
    }
    unsigned char* const xch = lowbit_xch + wave * (16 * kPitch);
    unsigned char* const xch_put = xch + (lane / kPiecesPerRow) * kPitch + (lane % kPiecesPerRow) * 16;  // + kRowsPerLoad j rows
    const unsigned char* const xch_get = xch + i * kPitch + q * (F::kCodes * 2);                        // + 16 c

    // constant A of the offset MFMA: row 0 = the offsets of the eight k of an MFMA (pairs 0..3 of the
    // lane's codes: the pattern repeats every byte, so every MFMA has the same), row 1 = ones
    uint32_t a_corr[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        if constexpr (DT == TPQ_DTYPE_F16) a_corr[h] = i == 0 ? F::magic(h) : i == 1 ? 0x3C003C00u : 0u;
        else a_corr[h] = (i == 0 && kFieldsInPlace) ? F::magic_bf(h) : i == 1 ? 0x3F803F80u : 0u;
    }
    uint32_t magic[F::kMagics];  // kept in VGPRs behind opaque moves: v_and_or_b32 takes one scalar operand
#pragma unroll
    for (int t = 0; t < F::kMagics; ++t) asm volatile("v_mov_b32 %0, %1" : "=v"(magic[t]) : "s"(DT == TPQ_DTYPE_F16 ? F::magic(t) : F::magic_bf(t)));

    struct Step {
        uint4 w[NB];     // kBytes of each are used
        uint4 p[NB][2];  // (scale, zero) of four channels
        uint4 xv[XL];    // as loaded: piece lane % kPiecesPerRow of row kRowsPerLoad j + lane / kPiecesPerRow
    };
    auto load = [&](int s, Step& st) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint8_t* src = w_base[b] + static_cast<size_t>(s) * (4 * F::kBytes);
            if constexpr (F::kBytes == 16) st.w[b] = nt_load(reinterpret_cast<const uint4*>(src));
            if constexpr (F::kBytes == 8) { const uint2 t = nt_load(reinterpret_cast<const uint2*>(src)); st.w[b] = make_uint4(t.x, t.y, 0, 0); }
            if constexpr (F::kBytes == 4) st.w[b] = make_uint4(nt_load(reinterpret_cast<const uint32_t*>(src)), 0, 0, 0);
            if constexpr (BITS == 8) st.w[b] = make_uint4(st.w[b].x ^ kSignFlip, st.w[b].y ^ kSignFlip, st.w[b].z ^ kSignFlip, st.w[b].w ^ kSignFlip);
            const uint4* prm = reinterpret_cast<const uint4*>(sz_base[b] + static_cast<size_t>(s >> group_shift) * N * 2);
            st.p[b][0] = prm[0];
            st.p[b][1] = prm[1];
        }
#pragma unroll
        for (int j = 0; j < XL; ++j) st.xv[j] = x_base[j][static_cast<size_t>(s) * kPiecesPerRow];
    };

    float yacc[NB][4];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) yacc[b][v] = 0.0f;
    auto compute = [&](const Step& st) {
        float4_t aux = {0.0f, 0.0f, 0.0f, 0.0f}, d[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) d[b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        // the step's activations into the exchange area and this lane's pieces out of it (LDS keeps a wavefront's
        // accesses in order: the reads of the step before are served before these writes)
#pragma unroll
        for (int j = 0; j < XL; ++j) *reinterpret_cast<uint4*>(xch_put + j * kRowsPerLoad * kPitch) = st.xv[j];
        uint4 xb[F::kCodes / 8];
#pragma unroll
        for (int c = 0; c < F::kCodes / 8; ++c) xb[c] = *reinterpret_cast<const uint4*>(xch_get + c * 16);
#pragma unroll
        for (int u = 0; u < F::kCodes / 8; ++u) {  // MFMA u (16x16x32): codes 8u .. 8u+7 of the lane
            const word4_t cv = {a_corr[0], a_corr[1], a_corr[2], a_corr[3]};
            const word4_t bv = {xb[u].x, xb[u].y, xb[u].z, xb[u].w};  // the same eight k of the activations
            if constexpr (DT == TPQ_DTYPE_F16) aux = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, cv), __builtin_bit_cast(half8_t, bv), aux, 0, 0, 0);
            else aux = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, cv), __builtin_bit_cast(bf8_t, bv), aux, 0, 0, 0);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                uint32_t a[4];
#pragma unroll
                for (int h = 0; h < 4; ++h) {
                    const int t = 4 * u + h;
                    const uint32_t word = dword_at(st.w[b], F::byte_lo(t) >> 2);
                    if constexpr (DT == TPQ_DTYPE_F16) {
                        const uint32_t both = __builtin_amdgcn_perm(0u, word, F::select(t));
                        a[h] = (both & F::mask(t)) | magic[t % F::kMagics];
                    } else if constexpr (kFieldsInPlace) {
                        const uint32_t both = __builtin_amdgcn_perm(word >> 1, word, F::select_bf(t));
                        a[h] = (both & F::mask_bf(t)) | magic[t % F::kMagics];
                    } else {
                        const float lo = static_cast<float>((word >> (8 * (F::byte_lo(t) & 3) + F::pos_lo(t))) & F::kField);
                        const float hi = static_cast<float>((word >> (8 * (F::byte_hi(t) & 3) + F::pos_hi(t))) & F::kField);
                        a[h] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo), 0x07060302u);
                    }
                }
                const word4_t av = {a[0], a[1], a[2], a[3]};
                if constexpr (DT == TPQ_DTYPE_F16) d[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, av), __builtin_bit_cast(half8_t, bv), d[b], 0, 0, 0);
                else d[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, av), __builtin_bit_cast(bf8_t, bv), d[b], 0, 0, 0);
            }
            // Without this the compiler expands the codes of all MFMAs of a step ahead of the first one; bfloat16 then
            // runs out of registers at three blocks of channels (scratch traffic).  fp16 stays within them, and the
            // fence helps it only with two activation loads per step (4096 -> 11008 at 8 rows, 1 / 2 / 4 bits:
            // 9.6 / 9.9 / 10.6 -> 9.0 / 9.7 / 10.2 us; at 2 and 4 rows it costs 0.2 - 0.4).
            if constexpr (kFieldsInPlace && (DT != TPQ_DTYPE_F16 || XL == 2)) __builtin_amdgcn_sched_barrier(0);
        }
        // rows 0 and 1 of the offset product sit in lanes 0..15, registers 0 and 1
        const float corr = __shfl(aux[0], i, kWave), sx = __shfl(aux[1], i, kWave);
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint4& pv = st.p[b][v >> 1];
                const float scale = __builtin_bit_cast(float, (v & 1) ? pv.z : pv.x);
                const float zero = __builtin_bit_cast(float, (v & 1) ? pv.w : pv.y) + (BITS == 8 ? 128.0f : 0.0f);
                yacc[b][v] = __builtin_fmaf(scale, (d[b][v] - corr) - zero * sx, yacc[b][v]);
            }
    };

    // this wavefront's steps: wave, wave + WAVES, ...; two in flight (three or four, as many as 180 registers hold,
    // so that K = 4096 would be one trip to memory per wavefront, were measured and lost at every width and row count:
    // 4096 -> 11008, 1 bit, 2 / 8 / 16 rows 8.2 / 9.6 / 10.5 -> 9.4 / 10.2 / 12.7 us; at 8 bits, where a step is 64 k, four in
    // flight leave registers for two blocks of channels only, a second round of workgroups: 8 rows 16.0 -> 22.7 us)
    Step s0 = {}, s1 = {};
    int s = wave;
    if (s < steps) load(s, s0);
    if (s + WAVES < steps) load(s + WAVES, s1);
    drain_vector_loads();  // exact waits inside the loop (4096 -> 11008 at 8 rows, 1 / 2 / 4 bits: 9.0 / 9.7 / 10.2 -> 8.5 / 9.3 / 9.8 us)
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

#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave][4 * b + v][lane] = yacc[b][v];
    __syncthreads();
    if (wave == 0 && row_live) {  // lane (m, q): channels n0 + 16 b + 4 q + v
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int n = n0 + 16 * b + 4 * q;
            if (n < N) {  // N % 4 == 0: all four channels exist
                float sum[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    sum[v] = 0.0f;
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) sum[v] += red[w][4 * b + v][lane];
                    if (bias != nullptr) sum[v] += bias[n + v];
                }
                const uint32_t lo = Elem<DT>::store(sum[0]) | (static_cast<uint32_t>(Elem<DT>::store(sum[1])) << 16);
                const uint32_t hi = Elem<DT>::store(sum[2]) | (static_cast<uint32_t>(Elem<DT>::store(sum[3])) << 16);
                *reinterpret_cast<uint2*>(y + static_cast<size_t>(i) * N + n) = make_uint2(lo, hi);
            }
        }
    }
}

// code k of row `row` (any bits, either bit order)
__device__ __forceinline__ int code_at(const uint8_t* row, int64_t k, int bits, int per_byte, bool lsb_first) {
    const int i = static_cast<int>(k % per_byte);
    const int shift = lsb_first ? i * bits : 8 - (i + 1) * bits;
    return (row[k / per_byte] >> shift) & ((1 << bits) - 1);
}

// Value of a code as the reference dequantizes it: unpack_intx ends in codes.to(int8) and _dequantize_intx converts
// that int8 to float (tensorplay/ao/quantization/intx_weight_only.py:62-80, 110-124), so at 8 bits a byte of 128 or
// more counts as byte - 256; narrower fields never reach the sign bit.
__device__ __forceinline__ float code_value(uint32_t code, int bits) {
    return bits == 8 ? static_cast<float>(static_cast<int>(static_cast<int8_t>(code))) : static_cast<float>(code);
}

// Any floating activation dtype and bit width, K % 8 == 0, group % 8 == 0, aligned rows: a wavefront owns
// four consecutive output channels and a slab of up to four activation rows; a lane takes eight consecutive k
// per turn (1 to 8 bytes of each weight row), forms (code - zero) * scale in fp32 as the reference does, fp32
// fma, one wavefront reduction at the end.
constexpr int kVecChannels = 4, kVecRows = 4;

template <int DT>
__global__ __launch_bounds__(256) void lowbit_vector_kernel(
    const typename Elem<DT>::storage* __restrict__ x, const uint8_t* __restrict__ packed, const float* __restrict__ sz,
    const float* __restrict__ bias, typename Elem<DT>::storage* __restrict__ y, int64_t M, int64_t N, int64_t K,
    int64_t group, int bits, int lsb_first) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int64_t n0 = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * kVecChannels, m0 = static_cast<int64_t>(blockIdx.y) * kVecRows;
    if (n0 >= N) return;
    const int rows = static_cast<int>(M - m0 < kVecRows ? M - m0 : kVecRows);
    const int per_byte = 8 / bits, bytes = 8 / per_byte;  // bytes holding eight codes: 1, 2, 4 or 8
    const int pb_shift = per_byte == 8 ? 3 : per_byte == 4 ? 2 : per_byte == 2 ? 1 : 0;
    const int64_t pitch = K >> pb_shift;
    const uint32_t field = (1u << bits) - 1u;
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
        const int64_t g = k / group;
#pragma unroll
        for (int c = 0; c < kVecChannels; ++c) {
            const int64_t n = n0 + c < N ? n0 + c : N - 1;  // channels past N: a valid row, result dropped
            const uint8_t* src = packed + n * pitch + (k >> pb_shift);
            uint64_t raw;
            if (bytes == 8) { const uint2 t = nt_load(reinterpret_cast<const uint2*>(src)); raw = t.x | (static_cast<uint64_t>(t.y) << 32); }
            else if (bytes == 4) raw = nt_load(reinterpret_cast<const uint32_t*>(src));
            else if (bytes == 2) raw = *reinterpret_cast<const uint16_t*>(src);
            else raw = *src;
            const float2 p = *reinterpret_cast<const float2*>(sz + (g * N + n) * 2);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int i = e & (per_byte - 1);  // per_byte is 1, 2, 4 or 8
                const int shift = 8 * (e >> pb_shift) + (lsb_first ? i * bits : 8 - (i + 1) * bits);
                const float wv = (code_value(static_cast<uint32_t>(raw >> shift) & field, bits) - p.y) * p.x;
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
            float total = wave_sum(acc[c][r]);
            if (lane == 0 && r < rows && n0 + c < N) {
                if (bias != nullptr) total += bias[n0 + c];
                y[(m0 + r) * N + n0 + c] = Elem<DT>::store(total);
            }
        }
}

// One workgroup per output channel n and slab of up to 8 activation rows.
template <int DT>
__global__ __launch_bounds__(256) void lowbit_generic_kernel(
    const typename Elem<DT>::storage* __restrict__ x, const uint8_t* __restrict__ packed, const float* __restrict__ sz,
    const float* __restrict__ bias, typename Elem<DT>::storage* __restrict__ y, int64_t M, int64_t N, int64_t K,
    int64_t group, int bits, int lsb_first) {
    __shared__ float red[8][256 / kWave];
    const int64_t n = blockIdx.x, m0 = static_cast<int64_t>(blockIdx.y) * 8;
    const int rows = static_cast<int>(M - m0 < 8 ? M - m0 : 8);
    const int per_byte = 8 / bits;
    const uint8_t* wr = packed + n * ((K + per_byte - 1) / per_byte);
    float acc[8];
#pragma unroll
    for (int b = 0; b < 8; ++b) acc[b] = 0.0f;
    for (int64_t k = threadIdx.x; k < K; k += 256) {
        const float* p = sz + ((k / group) * N + n) * 2;
        const float wv = (code_value(code_at(wr, k, bits, per_byte, lsb_first), bits) - p[1]) * p[0];
#pragma unroll
        for (int b = 0; b < 8; ++b)
            if (b < rows) acc[b] = __builtin_fmaf(wv, Elem<DT>::load(x[(m0 + b) * K + k]), acc[b]);
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const float v = wave_sum(acc[b]);
        if (lane == 0) red[b][wave] = v;
    }
    __syncthreads();
    if (threadIdx.x < rows) {
        const int b = threadIdx.x;
        float total = (red[b][0] + red[b][1]) + (red[b][2] + red[b][3]);
        if (bias != nullptr) total += bias[n];
        y[(m0 + b) * N + n] = Elem<DT>::store(total);
    }
}

// Dense [N, K] weight of `DT`: (float(code) - zero) * scale formed in fp32, then rounded once.
template <int DT>
__global__ __launch_bounds__(256) void lowbit_dequantize_kernel(const uint8_t* __restrict__ packed, const float* __restrict__ sz,
                                                                typename Elem<DT>::storage* __restrict__ out, int64_t N, int64_t K,
                                                                int64_t group, int bits, int lsb_first) {
    const int per_byte = 8 / bits;
    const int64_t pitch = (K + per_byte - 1) / per_byte;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < N * K;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t n = idx / K, k = idx - n * K;
        const float* p = sz + ((k / group) * N + n) * 2;
        out[idx] = Elem<DT>::store((code_value(code_at(packed + n * pitch, k, bits, per_byte, lsb_first != 0), bits) - p[1]) * p[0]);
    }
}

// The same for K % 8 == 0 and group % 8 == 0 with aligned rows: a thread takes eight consecutive k of one row, i.e.
// `bytes` = 1, 2, 4 or 8 packed bytes in one load, one (scale, zero) pair, and 16 (two-byte T) or 32 contiguous output
// bytes; a wavefront reads and writes contiguous runs of a row.
template <int DT>
__global__ __launch_bounds__(256) void lowbit_dequantize_vec_kernel(const uint8_t* __restrict__ packed, const float* __restrict__ sz,
                                                                    typename Elem<DT>::storage* __restrict__ out, int64_t N, int64_t K,
                                                                    int64_t group, int bits, int lsb_first) {
    using S = typename Elem<DT>::storage;
    const int per_byte = 8 / bits, bytes = 8 / per_byte;
    const int pb_shift = per_byte == 8 ? 3 : per_byte == 4 ? 2 : per_byte == 2 ? 1 : 0;
    const int64_t pitch = K >> pb_shift, per_row = K >> 3, total = N * per_row;
    const uint32_t mask = (1u << bits) - 1u;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t n = idx / per_row, k0 = (idx - n * per_row) * 8;
        const uint8_t* src = packed + n * pitch + (k0 >> pb_shift);
        uint64_t v;
        if (bytes == 8) v = *reinterpret_cast<const uint64_t*>(src);
        else if (bytes == 4) v = *reinterpret_cast<const uint32_t*>(src);
        else if (bytes == 2) v = *reinterpret_cast<const uint16_t*>(src);
        else v = *src;
        const float2 p = *reinterpret_cast<const float2*>(sz + ((k0 / group) * N + n) * 2);  // (scale, zero)
        S o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int field = i & (per_byte - 1);
            const int shift = 8 * (i >> pb_shift) + (lsb_first ? field * bits : 8 - (field + 1) * bits);
            const uint32_t code = static_cast<uint32_t>(v >> shift) & mask;
            o[i] = Elem<DT>::store((code_value(code, bits) - p.y) * p.x);
        }
        S* dst = out + n * K + k0;
        if constexpr (sizeof(S) == 2) {
            *reinterpret_cast<uint4*>(dst) = make_uint4(o[0] | (static_cast<uint32_t>(o[1]) << 16), o[2] | (static_cast<uint32_t>(o[3]) << 16),
                                                        o[4] | (static_cast<uint32_t>(o[5]) << 16), o[6] | (static_cast<uint32_t>(o[7]) << 16));
        } else {
            reinterpret_cast<float4*>(dst)[0] = make_float4(o[0], o[1], o[2], o[3]);
            reinterpret_cast<float4*>(dst)[1] = make_float4(o[4], o[5], o[6], o[7]);
        }
    }
}

// codes uint8 [rows, cols] -> packed [rows, pitch]: one thread per packed byte, tail fields zero
__global__ __launch_bounds__(256) void lowbit_pack_kernel(const uint8_t* __restrict__ codes, uint8_t* __restrict__ packed, int64_t rows,
                                                          int64_t cols, int bits, int lsb_first) {
    const int per_byte = 8 / bits;
    const int64_t pitch = (cols + per_byte - 1) / per_byte;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < rows * pitch;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t r = idx / pitch, b = idx - r * pitch;
        uint32_t value = 0;
        for (int i = 0; i < per_byte && b * per_byte + i < cols; ++i) {
            const int shift = lsb_first ? i * bits : 8 - (i + 1) * bits;
            value |= (codes[r * cols + b * per_byte + i] & ((1u << bits) - 1u)) << shift;
        }
        packed[idx] = static_cast<uint8_t>(value);
    }
}

__global__ __launch_bounds__(256) void lowbit_unpack_kernel(const uint8_t* __restrict__ packed, uint8_t* __restrict__ codes, int64_t rows,
                                                            int64_t cols, int bits, int lsb_first) {
    const int per_byte = 8 / bits;
    const int64_t pitch = (cols + per_byte - 1) / per_byte;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < rows * cols;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t r = idx / cols, c = idx - r * cols;
        codes[idx] = static_cast<uint8_t>(code_at(packed + r * pitch, c, bits, per_byte, lsb_first != 0));
    }
}

template <int DT, int BITS, bool LSB>
int launch_mfma(const void* x, const uint8_t* packed, const float* sz, const float* bias, void* out, int64_t M, int64_t N,
                int64_t K, int group_shift, hipStream_t s) {
    // wavefronts per workgroup: each takes every WAVES-th step, two in flight
    static const int forced = [] { const char* e = tuning_env("TPQ_LOWBIT_WAVES"); return e ? atoi(e) : 0; }();
    static const int forced_nb = [] { const char* e = tuning_env("TPQ_LOWBIT_NB"); return e ? atoi(e) : 0; }();
    const int64_t steps = K / Fields<BITS, LSB>::kStepK;
    // measured at 4096 -> 11008, one row, 2 bits: 4 waves 11.1 us, 8 waves 10.4 - 11.0 us, 16 waves 14.3 us
    const int waves = forced == 4 || forced == 8 ? forced : steps >= 16 ? 8 : 4;
    // blocks of 16 channels per workgroup (eight wavefronts only): as many as leave about one workgroup per compute unit
    int nb = 1;
    if (waves == 8) nb = forced_nb >= 1 && forced_nb <= 3 ? forced_nb : (N >= 10240 ? 3 : N > 4096 ? 2 : 1);
    constexpr int kRowsPerLoad = kWave / (Fields<BITS, LSB>::kStepK / 8);  // 4, or 8 at one code per byte
    constexpr int kFull = 16 / kRowsPerLoad;                               // loads of activations per step for 16 rows
    for (int64_t m0 = 0; m0 < M; m0 += 16) {
        const int rows = static_cast<int>(M - m0 < 16 ? M - m0 : 16);
        const dim3 grid(static_cast<unsigned>((N + 16 * nb - 1) / (16 * nb)));
        const uint16_t* xs = static_cast<const uint16_t*>(x) + m0 * K;
        uint16_t* ys = static_cast<uint16_t*>(out) + m0 * N;
        const int n = static_cast<int>(N), k = static_cast<int>(K);
        const int loads = (rows + kRowsPerLoad - 1) / kRowsPerLoad;  // loads of activations per step: 1, 2 or kFull
        const size_t xch = static_cast<size_t>(waves) * 16 * lowbit_x_pitch<BITS, LSB>();
#define TPQ_LB_MFMA(W, XLV, NBV) lowbit_mfma_kernel<DT, BITS, LSB, W, XLV, NBV><<<grid, W * kWave, xch, s>>>(xs, packed, sz, bias, ys, rows, n, k, group_shift)
#define TPQ_LB_MFMA_X(W, NBV)                                              \
    do {                                                                   \
        if (loads <= 1) TPQ_LB_MFMA(W, 1, NBV);                            \
        else if (loads <= 2) TPQ_LB_MFMA(W, 2, NBV);                       \
        else TPQ_LB_MFMA(W, kFull, NBV);                                   \
    } while (0)
        if (waves == 4) TPQ_LB_MFMA_X(4, 1);
        else if (nb == 3) TPQ_LB_MFMA_X(8, 3);
        else if (nb == 2) TPQ_LB_MFMA_X(8, 2);
        else TPQ_LB_MFMA_X(8, 1);
#undef TPQ_LB_MFMA_X
#undef TPQ_LB_MFMA
    }
    return check_launch("tpq_lowbit_mm (mfma)");
}

template <int DT>
int launch_generic(const void* x, const uint8_t* packed, const float* sz, const float* bias, void* out, int64_t M, int64_t N,
                   int64_t K, int64_t group, int bits, int lsb_first, hipStream_t s) {
    using S = typename Elem<DT>::storage;
    if (K > 0 && K % 8 == 0 && group % 8 == 0 && aligned(x, 32) && aligned(packed, 8) && aligned(sz, 8)) {
        const int64_t gx = (N + 4 * kVecChannels - 1) / (4 * kVecChannels), gy = (M + kVecRows - 1) / kVecRows;
        TPQ_REQUIRE(gx <= 0x7FFFFFFF && gy <= 65535, TPQ_ERR_INVALID_VALUE, "lowbit mm: shape too large");
        lowbit_vector_kernel<DT><<<dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)), 256, 0, s>>>(
            static_cast<const S*>(x), packed, sz, bias, static_cast<S*>(out), M, N, K, group, bits, lsb_first);
        return check_launch("tpq_lowbit_mm (vector)");
    }
    const int64_t slabs = (M + 7) / 8;
    TPQ_REQUIRE(N <= 0x7FFFFFFF && slabs <= 65535, TPQ_ERR_INVALID_VALUE, "lowbit mm: shape too large");
    lowbit_generic_kernel<DT><<<dim3(static_cast<unsigned>(N), static_cast<unsigned>(slabs)), 256, 0, s>>>(
        static_cast<const S*>(x), packed, sz, bias, static_cast<S*>(out), M, N, K, group, bits, lsb_first);
    return check_launch("tpq_lowbit_mm (generic)");
}

// One activation row (fp16 / bf16), 1, 2, 4 or (fp16) 8 bits: the packed rows are contiguous, so a wavefront reads them
// directly, as the one-row int8 weight-only kernel does.  A pass is 4096 k: lane l owns 64 of them, as TURNS
// segments of CPL codes (one 16-byte load each; 8 bytes at one bit), and the 128 bytes of activations that go with
// them, shared by the wavefront's four channels.  Every load is issued before the first use.  Per segment and channel
// y += scale (sum code x - zero sum x), a segment lying inside one group; three vector instructions per pair of codes.
// Workgroup = channel groups x passes; the lanes' sums meet by a butterfly, the passes' through LDS.
// CH channels per wavefront share a lane's 128 bytes of activations: 8 for large weights at 1 and 2 bits, where the
// activations re-read per wavefront would otherwise outweigh the packed bytes (8192 -> 28672 at 1 bit: 26.4 -> 21.9 us);
// 4 for small weights, which need the wavefronts (4096 x 4096 at 1 bit: 4.8 us against 6.0 with 8).

// The (scale, zero) pairs lie across the packed rows ([K / group][N] pairs): a lane asking for the pair of its segment
// and channel takes 8 bytes out of a cache line of its own, 128 lines per wavefront against 16 to 32 of packed weights.
// Parking them in LDS as well (the workgroup's channels are neighbours, so per group their pairs are one run; 16-byte
// pieces ahead of the weights, one more LDS-only barrier) was built and lost at every width (4096 -> 11008 at 1 / 2 / 4 /
// 8 bits: 6.4 / 6.7 / 7.8 / 11.5 -> 6.9 / 7.6 / 8.5 / 12.6 us): at these sizes every wavefront's loads arrive together and
// the 450 vector instructions of the three wavefronts a SIMD holds run one after the other behind the arrival, so the
// kernel is bound by that arithmetic and anything that sits between arrival and arithmetic adds to it.
// Fetching the pairs of two neighbouring channels with one 16-byte load (half the load instructions, the same lines)
// changed nothing either.
template <int DT, int BITS, bool LSB, int WAVES, int CH>
__global__ __launch_bounds__(WAVES * kWave) void lowbit_row_kernel(const uint16_t* __restrict__ x, const uint8_t* __restrict__ packed,
                                                                  const float* __restrict__ sz, const float* __restrict__ bias,
                                                                  uint16_t* __restrict__ y, int N, int K, int group, int passes, int groups) {
    constexpr int kLbRowChannels = CH;
    constexpr int kPerByte = 8 / BITS;
    constexpr int kLoadBytes = BITS == 1 ? 8 : 16;
    constexpr int kCpl = kLoadBytes * kPerByte;  // codes per load: 64, 64, 32, 16 (1, 2, 4, 8 bits)
    constexpr int kTurns = 64 / kCpl;            // 1, 1, 2, 4
    constexpr int kWords = kLoadBytes / 4;
    __shared__ float red[WAVES][kLbRowChannels];
    extern __shared__ __align__(16) unsigned char lb_row_x[];  // the activation row: chunk c of 16 bytes at 16 (c + c / 8)
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = wave / passes, pass = wave - g * passes;
    const int n0 = (blockIdx.x * groups + g) * kLbRowChannels;
    const bool active = g < groups && n0 < N;
    // The activations reach the lanes through LDS.  A lane owns runs of 64 consecutive k (128 bytes): asked for
    // directly, a wavefront load takes 16 bytes out of 64 cache lines, and the eight loads of a run are 512 line
    // look-ups per wavefront against 32 for the packed weights; the texture path's look-ups, not the bytes, were what
    // the kernel waited for.  The workgroup reads the row once, contiguously (a wavefront load = 1 KB = 8 lines),
    // and parks it with 16 bytes of padding per 128, so that the lanes' 16-byte reads spread over the banks.
    // Measured at 4096 -> 11008: 1 bit 7.15 -> 6.43 us, 2 bits 7.85 -> 6.86; 4 bits 7.84 -> 8.3 (a lane's runs are 64
    // bytes there, half the look-ups to save and twice the 16-byte LDS reads that collide), 8 bits no change: those two
    // keep the direct loads.
    constexpr bool kStageX = BITS <= 2;
    constexpr int kXRounds = 4;  // rounds of 16 bytes per thread in flight together
    constexpr int kXPerSweep = kXRounds * WAVES * kWave;
    const int x_chunks = K >> 3;
    typedef uint32_t words4 __attribute__((ext_vector_type(4)));
    const auto xg = pinned_global(reinterpret_cast<const words4*>(x));  // the loads stay here, ahead of the weights
    words4 xr[kXRounds];  // the first sweep is asked for here and parked behind the weights' requests
    if constexpr (kStageX) {
#pragma unroll
        for (int r = 0; r < kXRounds; ++r) {
            const int c = r * WAVES * kWave + static_cast<int>(threadIdx.x);
            xr[r] = xg[c < x_chunks ? c : 0];
        }
    }
    uint4 xv[kTurns][kCpl / 8];
    float acc[kLbRowChannels];
#pragma unroll
    for (int c = 0; c < kLbRowChannels; ++c) acc[c] = 0.0f;
    uint32_t wv[kLbRowChannels][kTurns][kWords];
    float2 p[kLbRowChannels][kTurns];
    bool live[kTurns];
    int k_first[kTurns];
    if (active) {
        const size_t pitch = static_cast<size_t>(K) / kPerByte;
#pragma unroll
        for (int t = 0; t < kTurns; ++t) {
            const int k0 = ((pass * kTurns + t) * kWave + lane) * kCpl;
            live[t] = k0 < K;
            const int kl = live[t] ? k0 : 0;  // past the end: a valid segment, multiplied by zeros
            k_first[t] = kl;
#pragma unroll
            for (int c = 0; c < kLbRowChannels; ++c) {
                const int n = n0 + c < N ? n0 + c : N - 1;
                const uint8_t* src = packed + static_cast<size_t>(n) * pitch + kl / kPerByte;
                if constexpr (kLoadBytes == 16) {
                    const uint4 q = nt_load(reinterpret_cast<const uint4*>(src));
                    wv[c][t][0] = q.x; wv[c][t][1] = q.y; wv[c][t][2] = q.z; wv[c][t][3] = q.w;
                } else {
                    const uint2 q = nt_load(reinterpret_cast<const uint2*>(src));
                    wv[c][t][0] = q.x; wv[c][t][1] = q.y;
                }
                p[c][t] = *reinterpret_cast<const float2*>(sz + (static_cast<size_t>(kl / group) * N + n) * 2);
            }
            if constexpr (!kStageX) {
                const uint4* xp = reinterpret_cast<const uint4*>(x + kl);
#pragma unroll
                for (int e = 0; e < kCpl / 8; ++e) xv[t][e] = live[t] ? xp[e] : make_uint4(0, 0, 0, 0);
            }
        }
    }
    if constexpr (kStageX) {
#pragma unroll
    for (int r = 0; r < kXRounds; ++r) {
        const int c = r * WAVES * kWave + static_cast<int>(threadIdx.x);
        if (c < x_chunks) *reinterpret_cast<words4*>(lb_row_x + 16 * (c + (c >> 3))) = xr[r];
    }
    for (int base = kXPerSweep; base < x_chunks; base += kXPerSweep) {  // long rows with few wavefronts
#pragma unroll
        for (int r = 0; r < kXRounds; ++r) {
            const int c = base + r * WAVES * kWave + static_cast<int>(threadIdx.x);
            xr[r] = xg[c < x_chunks ? c : 0];
        }
#pragma unroll
        for (int r = 0; r < kXRounds; ++r) {
            const int c = base + r * WAVES * kWave + static_cast<int>(threadIdx.x);
            if (c < x_chunks) *reinterpret_cast<words4*>(lb_row_x + 16 * (c + (c >> 3))) = xr[r];
        }
    }
    // the weights stay in flight across the barrier: it orders LDS traffic only
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    if (active) {
        if constexpr (kStageX) {
#pragma unroll
            for (int t = 0; t < kTurns; ++t)
#pragma unroll
                for (int e = 0; e < kCpl / 8; ++e) {
                    const int c = (k_first[t] >> 3) + e;
                    xv[t][e] = live[t] ? *reinterpret_cast<const uint4*>(lb_row_x + 16 * (c + (c >> 3))) : make_uint4(0, 0, 0, 0);
                }
        }
#pragma unroll
        for (int t = 0; t < kTurns; ++t)
#pragma unroll
            for (int c = 0; c < kLbRowChannels; ++c) {
                // the parameters enter the arithmetic here, not earlier: used ahead of the barrier they would be waited
                // for in front of it, and with them every load that was asked for before them
                if constexpr (kStageX) asm volatile("" : "+v"(p[c][t].x), "+v"(p[c][t].y));
                if constexpr (BITS == 8) {  // signed bytes: value + 128 in the fields, 128 more in the zero point
#pragma unroll
                    for (int w = 0; w < kWords; ++w) wv[c][t][w] ^= kSignFlip;
                    p[c][t].y += 128.0f;
                }
            }
        // Codes become 16-bit floats in place.  A field that lies at bit p of the mantissa of its 16-bit half, masked and
        // given the exponent under which bit p weighs one (one v_and_or_b32), is the pair (2^(kMant - p) + code,
        // 2^(kMant - p) + code') of the two halves' codes at that position; one v_dot2 multiplies it with the matching
        // pair of activations.  The kMant / BITS field positions inside the mantissa need no shift; one shift of the
        // word brings the next positions there.  The constants leave with the same pairs of activations multiplied by
        // the bare exponents, once per lane for all its channels:  y += scale ((dot - offsets) - zero sum x).
        // (One exponent for every position, each field shifted to the top of the mantissa first, was three
        // instructions per pair of codes instead of two and a shift per group of positions: 4096 -> 11008 at 1 / 2 bits
        // 6.6 / 6.8 -> 6.2 / 6.5 us, 8192 x 8192 8.0 / 8.5 -> 7.5 / 7.9, 8192 -> 28672 18.1 / 22.6 -> 16.3 / 20.2; 4 and 8 bits,
        // where a shift serves two positions or one, are unchanged.)
        using L = Lane16<DT>;
        constexpr int kMant = DT == TPQ_DTYPE_F16 ? 10 : 7, kExpBias = DT == TPQ_DTYPE_F16 ? 15 : 127;
        constexpr int kFieldsPerHalf = 16 / BITS;
        constexpr int kSpan = kMant / BITS < kFieldsPerHalf ? kMant / BITS : kFieldsPerHalf;  // positions served by one shift
        static_assert(kSpan >= 1, "a field fits the mantissa");
        constexpr int kShiftGroups = (kFieldsPerHalf + kSpan - 1) / kSpan;
        uint32_t magic[kSpan];  // kept in VGPRs behind an opaque move: v_and_or_b32 takes one literal only
#pragma unroll
        for (int i = 0; i < kSpan; ++i)
            asm volatile("v_mov_b32 %0, %1" : "=v"(magic[i]) : "s"((static_cast<uint32_t>(kExpBias + kMant - i * BITS) << kMant) * 0x00010001u));
#pragma unroll
        for (int t = 0; t < kTurns; ++t) {
            // activations: the natural pairs (k, k + 1) for the sum, and for every (word, position) the pair that
            // sits under the two halves of the word: codes e and e + 2 kPerByte of the segment
            auto half_of = [&](int e) -> uint32_t {
                const uint4& xq = xv[t][e >> 3];
                const uint32_t pair = ((e >> 1) & 3) == 0 ? xq.x : ((e >> 1) & 3) == 1 ? xq.y : ((e >> 1) & 3) == 2 ? xq.z : xq.w;
                return (e & 1) ? pair >> 16 : pair & 0xFFFFu;
            };
            float sx = 0.0f, off = 0.0f;
#pragma unroll
            for (int e = 0; e < kCpl; e += 2) sx = L::dot(half_of(e) | (half_of(e + 1) << 16), L::kOnes, sx);
            float s[kLbRowChannels];
#pragma unroll
            for (int c = 0; c < kLbRowChannels; ++c) s[c] = 0.0f;
#pragma unroll
            for (int w = 0; w < kWords; ++w)
#pragma unroll
                for (int sg = 0; sg < kShiftGroups; ++sg) {
                    uint32_t moved[kLbRowChannels];
#pragma unroll
                    for (int c = 0; c < kLbRowChannels; ++c) moved[c] = sg == 0 ? wv[c][t][w] : wv[c][t][w] >> (sg * kSpan * BITS);
#pragma unroll
                    for (int i = 0; i < kSpan; ++i) {
                        const int fp = sg * kSpan + i;  // field position inside a 16-bit half, from its low end
                        if (fp >= kFieldsPerHalf) continue;
                        const int byte = 4 * w + fp / kPerByte, pos = fp % kPerByte;
                        const int e = byte * kPerByte + (LSB ? pos : kPerByte - 1 - pos);
                        const uint32_t xpair = half_of(e) | (half_of(e + 2 * kPerByte) << 16);
                        const uint32_t mask = (((1u << BITS) - 1u) << (i * BITS)) * 0x00010001u;
                        off = L::dot(xpair, magic[i], off);
#pragma unroll
                        for (int c = 0; c < kLbRowChannels; ++c) s[c] = L::dot(xpair, (moved[c] & mask) | magic[i], s[c]);
                    }
                }
#pragma unroll
            for (int c = 0; c < kLbRowChannels; ++c)
                acc[c] = __builtin_fmaf(p[c][t].x, (s[c] - off) - p[c][t].y * sx, acc[c]);
        }
#pragma unroll
        for (int c = 0; c < kLbRowChannels; ++c) acc[c] = wave_sum(acc[c]);
    }
    if (lane == 0) {
#pragma unroll
        for (int c = 0; c < kLbRowChannels; ++c) red[wave][c] = acc[c];
    }
    __syncthreads();
    const int tid = threadIdx.x;
    if (tid < groups * kLbRowChannels) {  // thread = (group, channel): the passes in order
        const int gg = tid / kLbRowChannels, c = tid - gg * kLbRowChannels;
        const int n = (blockIdx.x * groups + gg) * kLbRowChannels + c;
        if (n < N) {
            float sum = 0.0f;
            for (int ps = 0; ps < passes; ++ps) sum += red[gg * passes + ps][c];
            if (bias != nullptr) sum += bias[n];
            y[n] = Elem<DT>::store(sum);
        }
    }
}

// false if the shape is not one the row kernel takes
template <int DT>
bool launch_lowbit_row(const void* x, const uint8_t* packed, const float* sz, const float* bias, void* out, int64_t N, int64_t K,
                       int64_t group, int bits, int lsb_first, bool forced, hipStream_t s, int* rc) {
    // 8 bits: fp16 only (a byte does not fit the 7 mantissa bits of bfloat16), workgroups of four or eight wavefronts
    // (four turns of loads per pass: 16 wavefronts would leave 128 registers per lane, too few), so K <= 32768
    if (bits != 1 && bits != 2 && bits != 4 && !(bits == 8 && DT == TPQ_DTYPE_F16)) return false;
    const int cpl = bits == 8 ? 16 : bits == 4 ? 32 : 64;
    if (K <= 0 || K % cpl != 0 || group % cpl != 0 || K > 65536 || N > 0x7FFFFFF0) return false;
    // Measured against the matrix-core kernel (us, 1 / 2 / 4 bits): 4096 -> 11008: 7.5 / 8.2 / 8.0 against 9.8 / 10.1 / 10.4;
    // 8192 x 8192: 9.6 / 10.7 / 10.9 against 12.7 / 13.2 / 15.4; 8192 -> 28672: 26.4 / 29.8 / 35.7 against 37.7 / 40.1 / 45.2;
    // 4096 x 4096: 4.8 / 5.0 / 4.7 against 4.8 / 5.1 / 5.2; 28672 -> 8192: 35.3 / 41.7 / 39.2 against 39.3 / 39.8 / 46.7.
    (void)forced;
    if (!aligned(x, 16) || !aligned(packed, 16) || !aligned(sz, 8) || !aligned(out, 2)) return false;
    const int passes = static_cast<int>((K + 4095) / 4096);
    // small weights need many workgroups to fill the chip: 4 wavefronts; 16 from 64 MB of packed bytes and for long rows
    int waves = (N * (K / (8 / bits)) >= (int64_t{1} << 26) || passes > 4) ? 16 : 4;
    if (bits == 8 && waves == 16) waves = 8;  // 8 bits: at most eight wavefronts (256 registers per lane)
    if (waves < passes) return false;
    const int groups = waves / passes, channels = (bits <= 2 && N * K >= (int64_t{1} << 26)) ? 8 : 4;
    const dim3 grid(static_cast<unsigned>((N + groups * channels - 1) / (groups * channels)));
    const auto* xp = static_cast<const uint16_t*>(x);
    auto* yp = static_cast<uint16_t*>(out);
    const int n = static_cast<int>(N), k = static_cast<int>(K), gr = static_cast<int>(group);
    const size_t x_lds = bits <= 2 ? (static_cast<size_t>(K) * 2 / 16) * 18 + 32 : 0;  // 16-byte chunks with 16 bytes of padding per eight
#define TPQ_LBROW_C(B, L, W, C)                                                                                               \
    do {                                                                                                                      \
        auto kernel = lowbit_row_kernel<DT, B, L, W, C>;                                                                      \
        static std::atomic<uint64_t> configured{0};                                                                           \
        if (x_lds > 48 * 1024)                                                                                                \
            if (int e = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), 160 * 1024 - 4096, configured, "lowbit mm")) { \
                *rc = e;                                                                                                      \
                return true;                                                                                                  \
            }                                                                                                                 \
        kernel<<<grid, W * kWave, x_lds, s>>>(xp, packed, sz, bias, yp, n, k, gr, passes, groups);                            \
    } while (0)
#define TPQ_LBROW(B, L, W) do { if (B <= 2 && channels == 8) TPQ_LBROW_C(B, L, W, (B <= 2 ? 8 : 4)); else TPQ_LBROW_C(B, L, W, 4); } while (0)
#define TPQ_LBROW_W(B, L) do { if (waves == 4) TPQ_LBROW(B, L, 4); else TPQ_LBROW(B, L, 16); } while (0)
#define TPQ_LBROW_L(B) do { if (lsb_first) TPQ_LBROW_W(B, true); else TPQ_LBROW_W(B, false); } while (0)
    if (bits == 1) TPQ_LBROW_L(1); else if (bits == 2) TPQ_LBROW_L(2); else if (bits == 4) TPQ_LBROW_L(4);
    else if constexpr (DT == TPQ_DTYPE_F16) { if (waves == 4) TPQ_LBROW(8, true, 4); else TPQ_LBROW(8, true, 8); }  // one code per byte: the bit order does not matter
#undef TPQ_LBROW_L
#undef TPQ_LBROW_W
#undef TPQ_LBROW
#undef TPQ_LBROW_C
    *rc = check_launch("tpq_lowbit_mm (row)");
    return true;
}

int check_lowbit(const char* op, int bits, int lsb_first, int64_t N, int64_t K, int64_t group) {
    TPQ_REQUIRE(bits >= 1 && bits <= 8, TPQ_ERR_INVALID_VALUE, "%s: bits must be in [1, 8], got %d", op, bits);
    TPQ_REQUIRE(lsb_first == 0 || lsb_first == 1, TPQ_ERR_INVALID_VALUE, "%s: lsb_first must be 0 or 1", op);
    TPQ_REQUIRE(N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "%s: negative shape", op);
    TPQ_REQUIRE(group > 0 && K % group == 0, TPQ_ERR_INVALID_VALUE, "%s: K=%lld must be divisible by groupsize=%lld", op,
                static_cast<long long>(K), static_cast<long long>(group));
    return TPQ_OK;
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int tpq_lowbit_mm(const void* x, int dtype, int64_t M, int64_t K, const uint8_t* packed, int bits,
                             int lsb_first, int64_t N, int64_t group, const float* scales_and_zeros, const float* bias,
                             void* out, void* stream) {
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F32 || dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16, TPQ_ERR_INVALID_TYPE,
                "lowbit mm: activations must be floating point");
    TPQ_REQUIRE(M >= 0, TPQ_ERR_INVALID_VALUE, "lowbit mm: negative shape");
    if (int rc = check_lowbit("lowbit mm", bits, lsb_first, N, K, group)) return rc;
    if (M == 0 || N == 0) return TPQ_OK;
    TPQ_REQUIRE(out != nullptr, TPQ_ERR_INVALID_VALUE, "lowbit mm: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    // K = 0 is an empty sum: the plain kernel then writes the bias (or zeros) and reads nothing else
    TPQ_REQUIRE(K == 0 || (x && packed && scales_and_zeros), TPQ_ERR_INVALID_VALUE, "lowbit mm: null pointer");
    const int per_byte = 8 / bits;
    const int step_k = per_byte >= 2 ? 128 : 64;
    int group_shift = -1;
    if (group % step_k == 0) {
        const int64_t per_group = group / step_k;
        if ((per_group & (per_group - 1)) == 0) {
            group_shift = 0;
            while ((int64_t{1} << group_shift) < per_group) ++group_shift;
        }
    }
    const bool fast = dtype != TPQ_DTYPE_F32 && K > 0 && group_shift >= 0 && K % step_k == 0 && N % 4 == 0 && K <= 0x7FFFFF80 &&
                      N <= 0x7FFFFFF0 && aligned(x, 16) && aligned(packed, 16) && aligned(scales_and_zeros, 16) && aligned(out, 8);
    const int forced_row = route_override_lowbit_row();
    if (M == 1 && dtype != TPQ_DTYPE_F32 && forced_row != 0) {  // a test-hook build pins the route: never / wherever the shape allows
        int rc = TPQ_OK;
        if (dtype == TPQ_DTYPE_F16 ? launch_lowbit_row<TPQ_DTYPE_F16>(x, packed, scales_and_zeros, bias, out, N, K, group, bits, lsb_first, forced_row == 1, s, &rc)
                                   : launch_lowbit_row<TPQ_DTYPE_BF16>(x, packed, scales_and_zeros, bias, out, N, K, group, bits, lsb_first, forced_row == 1, s, &rc))
            return rc;
    }
    if (fast) {
#define TPQ_LB_CASE(BITS)                                                                                                      \
    case BITS:                                                                                                                 \
        if (dtype == TPQ_DTYPE_F16)                                                                                            \
            return lsb_first ? launch_mfma<TPQ_DTYPE_F16, BITS, true>(x, packed, scales_and_zeros, bias, out, M, N, K, group_shift, s) \
                             : launch_mfma<TPQ_DTYPE_F16, BITS, false>(x, packed, scales_and_zeros, bias, out, M, N, K, group_shift, s); \
        return lsb_first ? launch_mfma<TPQ_DTYPE_BF16, BITS, true>(x, packed, scales_and_zeros, bias, out, M, N, K, group_shift, s) \
                         : launch_mfma<TPQ_DTYPE_BF16, BITS, false>(x, packed, scales_and_zeros, bias, out, M, N, K, group_shift, s);
        switch (bits) {
            TPQ_LB_CASE(1)
            TPQ_LB_CASE(2)
            TPQ_LB_CASE(3)
            TPQ_LB_CASE(4)
            TPQ_LB_CASE(5)
            TPQ_LB_CASE(6)
            TPQ_LB_CASE(7)
            TPQ_LB_CASE(8)
        }
#undef TPQ_LB_CASE
    }
    switch (dtype) {
        case TPQ_DTYPE_F32: return launch_generic<TPQ_DTYPE_F32>(x, packed, scales_and_zeros, bias, out, M, N, K, group, bits, lsb_first, s);
        case TPQ_DTYPE_F16: return launch_generic<TPQ_DTYPE_F16>(x, packed, scales_and_zeros, bias, out, M, N, K, group, bits, lsb_first, s);
        default: return launch_generic<TPQ_DTYPE_BF16>(x, packed, scales_and_zeros, bias, out, M, N, K, group, bits, lsb_first, s);
    }
}

TPQ_EXPORT int tpq_lowbit_dequantize(const uint8_t* packed, int bits, int lsb_first, int64_t N, int64_t K, int64_t group,
                                     const float* scales_and_zeros, int dtype, void* out, void* stream) {
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F32 || dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16, TPQ_ERR_INVALID_TYPE,
                "lowbit dequantize: the dense weight must be floating point");
    if (int rc = check_lowbit("lowbit dequantize", bits, lsb_first, N, K, group)) return rc;
    if (N == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(packed && scales_and_zeros && out, TPQ_ERR_INVALID_VALUE, "lowbit dequantize: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (K % 8 == 0 && group % 8 == 0 && aligned(packed, 8) && aligned(scales_and_zeros, 8) && aligned(out, 16)) {
        const int64_t vblocks = (N * (K / 8) + 255) / 256;
        const unsigned vgrid = static_cast<unsigned>(vblocks > (1 << 22) ? (1 << 22) : vblocks);
        switch (dtype) {
            case TPQ_DTYPE_F32:
                lowbit_dequantize_vec_kernel<TPQ_DTYPE_F32><<<vgrid, 256, 0, s>>>(packed, scales_and_zeros, static_cast<float*>(out), N, K, group, bits, lsb_first);
                break;
            case TPQ_DTYPE_F16:
                lowbit_dequantize_vec_kernel<TPQ_DTYPE_F16><<<vgrid, 256, 0, s>>>(packed, scales_and_zeros, static_cast<uint16_t*>(out), N, K, group, bits, lsb_first);
                break;
            default:
                lowbit_dequantize_vec_kernel<TPQ_DTYPE_BF16><<<vgrid, 256, 0, s>>>(packed, scales_and_zeros, static_cast<uint16_t*>(out), N, K, group, bits, lsb_first);
                break;
        }
        return check_launch("tpq_lowbit_dequantize");
    }
    const int64_t blocks = (N * K + 255) / 256;
    const unsigned grid = static_cast<unsigned>(blocks > (1 << 20) ? (1 << 20) : blocks);
    switch (dtype) {
        case TPQ_DTYPE_F32:
            lowbit_dequantize_kernel<TPQ_DTYPE_F32><<<grid, 256, 0, s>>>(packed, scales_and_zeros, static_cast<float*>(out), N, K, group, bits, lsb_first);
            break;
        case TPQ_DTYPE_F16:
            lowbit_dequantize_kernel<TPQ_DTYPE_F16><<<grid, 256, 0, s>>>(packed, scales_and_zeros, static_cast<uint16_t*>(out), N, K, group, bits, lsb_first);
            break;
        default:
            lowbit_dequantize_kernel<TPQ_DTYPE_BF16><<<grid, 256, 0, s>>>(packed, scales_and_zeros, static_cast<uint16_t*>(out), N, K, group, bits, lsb_first);
            break;
    }
    return check_launch("tpq_lowbit_dequantize");
}

TPQ_EXPORT int tpq_lowbit_pack(const uint8_t* codes, int bits, int lsb_first, int64_t rows, int64_t cols, uint8_t* packed, void* stream) {
    if (int rc = check_lowbit("lowbit pack", bits, lsb_first, rows, cols, 1)) return rc;
    if (rows == 0 || cols == 0) return TPQ_OK;
    TPQ_REQUIRE(codes && packed, TPQ_ERR_INVALID_VALUE, "lowbit pack: null pointer");
    const int per_byte = 8 / bits;
    const int64_t blocks = (rows * ((cols + per_byte - 1) / per_byte) + 255) / 256;
    lowbit_pack_kernel<<<static_cast<unsigned>(blocks > (1 << 20) ? (1 << 20) : blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
        codes, packed, rows, cols, bits, lsb_first);
    return check_launch("tpq_lowbit_pack");
}

TPQ_EXPORT int tpq_lowbit_unpack(const uint8_t* packed, int bits, int lsb_first, int64_t rows, int64_t cols, uint8_t* codes, void* stream) {
    if (int rc = check_lowbit("lowbit unpack", bits, lsb_first, rows, cols, 1)) return rc;
    if (rows == 0 || cols == 0) return TPQ_OK;
    TPQ_REQUIRE(codes && packed, TPQ_ERR_INVALID_VALUE, "lowbit unpack: null pointer");
    const int64_t blocks = (rows * cols + 255) / 256;
    lowbit_unpack_kernel<<<static_cast<unsigned>(blocks > (1 << 20) ? (1 << 20) : blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
        packed, codes, rows, cols, bits, lsb_first);
    return check_launch("tpq_lowbit_unpack");
}
