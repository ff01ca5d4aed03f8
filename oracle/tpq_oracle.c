/*
 * CPU oracle for the quantized-linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic of the reference's
 * CPU (and, for the device-only layouts, device) quantized kernels so that
 * the HIP kernels can be checked against it bit for bit (integers) or within
 * a stated tolerance (floating point).  Nothing in the shipped library links
 * or calls it: only tests/, the smoke check and the benchmark's cpu_baseline
 * leg load the shared object built from this file.
 *
 * Every function names the reference lines (relative to the reference root)
 * it follows.  Parity status of each function is listed next to it as
 * "pinned by": the independent evidence the test-suite checks it against.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; fused multiply-adds
 * appear only where the reference itself asks for one, via fmaf()).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2 };

/* ------------------------------------------------------------------------ */
/* 16-bit float conversions                                                  */
/* ------------------------------------------------------------------------ */

/* bf16 -> f32 is a shift; f32 -> bf16 rounds to nearest even and quiets NaN
 * (p10/include/BFloat16.h:100-111). */
static inline float bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu) != 0) return 0x7FC0u;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* IEEE binary16 <-> binary32, round to nearest even (the reference's Half
 * converts through float the same way, p10/include/Half.h:166-181). */
static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else {
            int e = -1;
            do { man <<= 1; ++e; } while (!(man & 0x400u));
            man &= 0x3FFu;
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7F800000u | (man << 13);
    } else {
        u = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t f32_to_f16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t absu = u & 0x7FFFFFFFu;
    if (absu >= 0x7F800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (absu > 0x7F800000u ? 0x200u : 0));
    }
    if (absu >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absu < 0x38800000u) { /* subnormal half or zero */
        if (absu < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
        int shift = 126 - (int)(absu >> 23); /* 14..24 */
        uint32_t man = (absu & 0x7FFFFFu) | 0x800000u;
        uint32_t lsb = 1u << shift;
        uint32_t half = lsb >> 1;
        uint32_t q = man >> shift;
        uint32_t rem = man & (lsb - 1);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
    uint32_t rebased = absu - 0x38000000u; /* exponent 127 -> 15 */
    uint32_t q = rebased >> 13;
    uint32_t rem = rebased & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
}

static inline float load_as_f32(const void* p, int dtype, int64_t i) {
    switch (dtype) {
        case ORC_F16: return f16_to_f32(((const uint16_t*)p)[i]);
        case ORC_BF16: return bf16_to_f32(((const uint16_t*)p)[i]);
        default: return ((const float*)p)[i];
    }
}

static inline void store_from_f32(void* p, int dtype, int64_t i, float v) {
    switch (dtype) {
        case ORC_F16: ((uint16_t*)p)[i] = f32_to_f16(v); break;
        case ORC_BF16: ((uint16_t*)p)[i] = f32_to_bf16(v); break;
        default: ((float*)p)[i] = v; break;
    }
}

/* Round a float through the storage type T and back (one "T operation"). */
static inline float round_through(float v, int dtype) {
    switch (dtype) {
        case ORC_F16: return f16_to_f32(f32_to_f16(v));
        case ORC_BF16: return bf16_to_f32(f32_to_bf16(v));
        default: return v;
    }
}

ORC_API void orc_convert(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n) {
    for (int64_t i = 0; i < n; ++i) store_from_f32(dst, dst_dtype, i, load_as_f32(src, src_dtype, i));
}

/* ------------------------------------------------------------------------ */
/* A1 / A2 / N7: row-wise signed quantizer                                   */
/* ------------------------------------------------------------------------ */

/*
 * Follows rowwise_quantize_cpu_impl (p10/include/QuantNativeImpl.h:1162-1187)
 * and its low-bit twin lowbit_quantize_cpu_impl
 * (p10/src/backend/cpu/LowBitGemmKernels.cpp:19-52):
 *   absmax = max_k |float(x)|            (fp32, starting from 0)
 *   scale  = max(absmax, eps) / divisor  (fp32 divide)
 *   code   = clamp(nearbyint(float(x) / scale), qmin, qmax)   (ties to even)
 *   sign_mode: code = x >= 0 ? qmax : qmin
 * int8: divisor 127, range [-127,127]; int4: 7, [-8,7]; int2: 2, [-2,1];
 * binary: 1, sign mode.
 * Pinned by: numpy float32 closed form, torch.round(x/scale), invariants
 * (tests/test_oracle_quantize.py).
 */
ORC_API void orc_quantize_rowwise(const void* x, int dtype, int64_t M, int64_t K, float eps,
                                  float divisor, int qmin, int qmax, int sign_mode,
                                  int8_t* codes, float* scales) {
    for (int64_t r = 0; r < M; ++r) {
        float absmax = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
            float a = fabsf(load_as_f32(x, dtype, r * K + k));
            /* std::max(absmax, a): keeps absmax when a is NaN */
            absmax = (absmax < a) ? a : absmax;
        }
        const float scale = ((absmax < eps) ? eps : absmax) / divisor;
        scales[r] = scale;
        for (int64_t k = 0; k < K; ++k) {
            const float v = load_as_f32(x, dtype, r * K + k);
            int c;
            if (sign_mode) {
                c = (v >= 0.0f) ? qmax : qmin;
            } else {
                c = (int)nearbyintf(v / scale);
                c = c < qmin ? qmin : (c > qmax ? qmax : c);
            }
            codes[r * K + k] = (int8_t)c;
        }
    }
}

/* ------------------------------------------------------------------------ */
/* A3: integer matrix product                                                */
/* ------------------------------------------------------------------------ */

/*
 * Follows int_mm_loop (p10/src/backend/cpu/IntMM.cpp:36-57): C[M,N] int32 =
 * A[M,K] (int8 or uint8) x B[K,N] int8, i-k-j walk, rows of A that hold a
 * zero skip the inner loop.  ldb/ldn let the caller hand over either a
 * contiguous [K,N] operand (b_stride_k = N, b_stride_n = 1) or the
 * transposed view of a [N,K] weight (b_stride_k = 1, b_stride_n = K), which
 * is how the reference's Python passes it (int8_mixed_precision.py:69).
 * Pinned by: widened numpy product, torch._int_mm on CPU.
 */
ORC_API void orc_int_mm(const void* a, int a_unsigned, const int8_t* b, int64_t b_stride_k,
                        int64_t b_stride_n, int32_t* c, int64_t M, int64_t K, int64_t N) {
    for (int64_t i = 0; i < M; ++i) {
        int32_t* row = c + i * N;
        memset(row, 0, sizeof(int32_t) * (size_t)N);
        for (int64_t k = 0; k < K; ++k) {
            const int32_t s = a_unsigned ? (int32_t)((const uint8_t*)a)[i * K + k]
                                         : (int32_t)((const int8_t*)a)[i * K + k];
            if (s == 0) continue;
            const int8_t* brow = b + k * b_stride_k;
            if (b_stride_n == 1) {
                for (int64_t j = 0; j < N; ++j) row[j] += s * (int32_t)brow[j];
            } else {
                for (int64_t j = 0; j < N; ++j) row[j] += s * (int32_t)brow[j * b_stride_n];
            }
        }
    }
}

/* Same product for a [N,K] weight, dot-product walk (cache friendly for the
 * benchmark's CPU baseline; integer sums are order independent, so the result
 * is identical to orc_int_mm with b_stride_k = 1, b_stride_n = K). */
ORC_API void orc_int_mm_nk(const int8_t* a, const int8_t* w, int32_t* c, int64_t M, int64_t K,
                           int64_t N, int64_t row_begin, int64_t row_end) {
    for (int64_t i = row_begin; i < row_end && i < M; ++i) {
        const int8_t* ar = a + i * K;
        for (int64_t j = 0; j < N; ++j) {
            const int8_t* wr = w + j * K;
            int32_t s = 0;
            for (int64_t k = 0; k < K; ++k) s += (int32_t)ar[k] * (int32_t)wr[k];
            c[i * N + j] = s;
        }
    }
}

/* ------------------------------------------------------------------------ */
/* A4: per-row x per-column rescale                                          */
/* ------------------------------------------------------------------------ */

/*
 * Follows _int8_mm_rescale_cpu (p10/include/QuantNativeImpl.h:1240-1264) and
 * the device kernel (p10/src/backend/cuda/QuantGemmKernels.cu:1611-1623):
 * res = (float(acc) * rs[r]) * cs[c], two fp32 multiplies in that order.
 * out_dtype other than F32 rounds that fp32 value once (the fused epilogue's
 * bf16/fp16 store); bias, when given, is added in fp32 before the rounding
 * (the reference adds it afterwards in Python, int8_mixed_precision.py:242).
 * Pinned by: numpy float32 closed form; scaled_int8_mm vs float matmul
 * (test/quantization/test_int8_mixed_precision.py:219-229).
 */
ORC_API void orc_int8_mm_rescale(const int32_t* acc, const float* rs, const float* cs,
                                 const float* bias, void* out, int out_dtype, int64_t M,
                                 int64_t N) {
    for (int64_t r = 0; r < M; ++r) {
        const float sr = rs[r];
        for (int64_t c = 0; c < N; ++c) {
            float v = (float)acc[r * N + c] * sr;
            v = v * cs[c];
            if (bias) v = v + bias[c];
            store_from_f32(out, out_dtype, r * N + c, v);
        }
    }
}

/* ------------------------------------------------------------------------ */
/* A6': CPU int4 packed layout                                               */
/* ------------------------------------------------------------------------ */

/*
 * Follows int4_pack_impl (p10/src/backend/cpu/QuantizedElementwiseKernels.cpp
 * :370-390).  `columns` is 4 x the float vector width of the ISA tier the
 * reference was built for (64 on AVX-512, 32 on AVX2 and on the plain tier,
 * :19); `half_split` is 1 on the two vector tiers (full blocks pair column
 * `lane` with `lane + columns/2`) and 0 on the plain tier (always pairs
 * 2*lane with 2*lane+1).  Tail blocks always use the adjacent pairing.
 * Pinned by: byte equality with torch._convert_weight_to_int4pack_for_cpu
 * (columns=64, half_split=1 on this AVX-512 host), the same check the
 * reference makes (test/quantization/test_native_operator_families.py:587-589).
 */
ORC_API void orc_int4_pack_cpu(const int32_t* codes, uint8_t* dst, int64_t n, int64_t k,
                               int columns, int half_split) {
    const int64_t blocks = (n + columns - 1) / columns;
    for (int64_t block = 0; block < blocks; ++block) {
        const int64_t first = block * columns;
        const int64_t width = (n - first < columns) ? (n - first) : columns;
        const int full = half_split && width == columns;
        for (int64_t feature = 0; feature < k; ++feature) {
            for (int64_t lane = 0; lane < width / 2; ++lane) {
                const int64_t lo = full ? lane : lane * 2;
                const int64_t hi = full ? lane + width / 2 : lane * 2 + 1;
                dst[first * k / 2 + feature * width / 2 + lane] =
                    (uint8_t)((uint8_t)codes[(first + lo) * k + feature] |
                              (uint8_t)((uint8_t)codes[(first + hi) * k + feature] << 4));
            }
        }
    }
}

/* Code of (column, feature) inside the CPU layout (inverse of the above). */
static inline int cpu_layout_code(const uint8_t* packed, int64_t n, int64_t k, int columns,
                                  int half_split, int64_t col, int64_t feature) {
    const int64_t first = col / columns * columns;
    const int64_t width = (n - first < columns) ? (n - first) : columns;
    const int64_t c = col - first;
    const int full = half_split && width == columns;
    const int64_t byte = full ? c % (width / 2) : c / 2;
    const int shift = full ? (c >= width / 2) * 4 : (int)(c % 2) * 4;
    return (packed[first * k / 2 + feature * width / 2 + byte] >> shift) & 15;
}

/*
 * A7': follows int4_mm_codes (QuantizedElementwiseKernels.cpp:392-507): for
 * each output, fp32 sequential over k:  w = fma(code-8, scale, zero);
 * acc = fma(x, w, acc); result cast to the activation dtype.  scale/zero are
 * params[(k/group, n, {0,1})] in the activation dtype.  Every vector tile of
 * the reference (generic, AVX-512 bf16 rows :510-560) performs this same
 * per-output sequence; only the AVX2 bf16 tile folds -8*scale into the zero
 * first (:587) and is not modelled.
 * Pinned by: torch._weight_int4pack_mm_for_cpu (max error 0 in the
 * reference's own record benchmark/quantized_native_performance.json), fp64
 * dense product of the dequantised weight.
 */
ORC_API void orc_int4_mm_cpu(const void* x, int dtype, const uint8_t* packed, const void* params,
                             void* out, int64_t m, int64_t n, int64_t k, int64_t group,
                             int columns, int half_split, int64_t row_begin, int64_t row_end) {
    for (int64_t r = row_begin; r < row_end && r < m; ++r) {
        for (int64_t c = 0; c < n; ++c) {
            float acc = 0.0f;
            for (int64_t f = 0; f < k; ++f) {
                const int64_t g = f / group;
                const float scale = load_as_f32(params, dtype, (g * n + c) * 2);
                const float zero = load_as_f32(params, dtype, (g * n + c) * 2 + 1);
                const float code = (float)(cpu_layout_code(packed, n, k, columns, half_split, c, f) - 8);
                const float w = fmaf(code, scale, zero);
                acc = fmaf(load_as_f32(x, dtype, r * k + f), w, acc);
            }
            store_from_f32(out, dtype, r * n + c, acc);
        }
    }
}

/*
 * The same kernel as orc_int4_mm_cpu, organised like the reference's task
 * split (4 rows x one block of 64 columns per task, k outermost inside a
 * task; QuantizedElementwiseKernels.cpp:402-479) so that the compiler can
 * vectorise across the 64 columns.  Used as the timed CPU baseline; callers
 * spread column blocks over threads the way parallel_for spreads tasks.
 * AVX-512 layout only (columns = 64, half split), n % 64 == 0.  Every output
 * sees the identical fmaf sequence, so results equal orc_int4_mm_cpu bit for
 * bit (asserted in tests/test_oracle_int4.py).
 */
ORC_API void orc_int4_mm_cpu_blocked(const void* x, int dtype, const uint8_t* packed,
                                     const void* params, void* out, int64_t m, int64_t n,
                                     int64_t k, int64_t group, int64_t block_begin,
                                     int64_t block_end) {
    enum { C = 64, H = 32 };
    float* xf = (float*)malloc(sizeof(float) * (size_t)(m * k > 0 ? m * k : 1));
    for (int64_t i = 0; i < m * k; ++i) xf[i] = load_as_f32(x, dtype, i);
    for (int64_t block = block_begin; block < block_end; ++block) {
        const int64_t first = block * C;
        const uint8_t* wp = packed + first * k / 2;
        for (int64_t row = 0; row < m; row += 4) {
            const int rows = (int)(m - row < 4 ? m - row : 4);
            float acc[4][C];
            float scale[C], zero[C];
            for (int r = 0; r < 4; ++r)
                for (int c = 0; c < C; ++c) acc[r][c] = 0.0f;
            for (int64_t f = 0; f < k; ++f) {
                if (f % group == 0) {
                    const int64_t g = f / group;
                    for (int c = 0; c < C; ++c) {
                        scale[c] = load_as_f32(params, dtype, (g * n + first + c) * 2);
                        zero[c] = load_as_f32(params, dtype, (g * n + first + c) * 2 + 1);
                    }
                }
                const uint8_t* bytes = wp + f * H;
                float w[C];
                for (int lane = 0; lane < H; ++lane) {
                    const int b = bytes[lane];
                    w[lane] = fmaf((float)((b & 15) - 8), scale[lane], zero[lane]);
                    w[lane + H] = fmaf((float)((b >> 4) - 8), scale[lane + H], zero[lane + H]);
                }
                for (int r = 0; r < rows; ++r) {
                    const float a = xf[(row + r) * k + f];
                    for (int c = 0; c < C; ++c) acc[r][c] = fmaf(a, w[c], acc[r][c]);
                }
            }
            for (int r = 0; r < rows; ++r)
                for (int c = 0; c < C; ++c) store_from_f32(out, dtype, (row + r) * n + first + c, acc[r][c]);
        }
    }
    free(xf);
}

/* ------------------------------------------------------------------------ */
/* A6: device int4 packed layout                                             */
/* ------------------------------------------------------------------------ */

/*
 * Two stages, as the reference does it on the device
 * (p10/src/backend/cuda/QuantGemmKernels.cu:1349-1408):
 *  stage 1 (int4_pack_kernel, :322-330): byte e of [N, K/2] =
 *           (codes[2e+1] & 15) | (codes[2e] & 15) << 4  (even k in the HIGH nibble);
 *  stage 2 (matrix_to_m16n8k16_Bint4_layout<I>, :838-877): int32
 *           out[nTile][kOuter][t][i/2], t in 0..31, n = 8*nTile + t/4,
 *           four bytes ks = {b0, b0+4, b0+8, b0+12} + t%4 with
 *           b0 = (kOuter*I + i) * 8; rows or bytes out of range read as 0.
 *           word = lo(v3)<<28 | lo(v2)<<24 | lo(v1)<<20 | lo(v0)<<16 |
 *                  hi(v3)<<12 | hi(v2)<<8  | hi(v1)<<4  | hi(v0).
 * out has ceil(N/8) * ceil(K/(16 I)) * 32 * (I/2) words.
 * Pinned by: orc_int4_tc_dequantize below being its inverse (the reference's
 * two kernels are mutual inverses), and a direct nibble formula in numpy
 * (tests/test_oracle_int4.py).  No library twin runs on a CPU.
 */
ORC_API void orc_int4_pack_tc(const int32_t* codes, int64_t N, int64_t K, int inner,
                              int32_t* out) {
    const int64_t cols = K / 2; /* bytes per row after stage 1 */
    uint8_t* bytes = (uint8_t*)malloc((size_t)(N * cols > 0 ? N * cols : 1));
    for (int64_t e = 0; e < N * cols; ++e) {
        const int32_t low = codes[2 * e + 1] & 0x0f;
        const int32_t high = codes[2 * e] & 0x0f;
        bytes[e] = (uint8_t)(low | (high << 4));
    }
    const int64_t nTiles = (N + 7) / 8;
    const int64_t kSuper = (K + inner * 16 - 1) / (inner * 16);
    for (int64_t nTile = 0; nTile < nTiles; ++nTile)
        for (int64_t kOuter = 0; kOuter < kSuper; ++kOuter)
            for (int t = 0; t < 32; ++t)
                for (int i = 0; i < inner; i += 2) {
                    const int64_t n0 = nTile * 8 + t / 4;
                    const int64_t b0 = (kOuter * inner + i) * 8;
                    const int64_t ks[4] = {b0 + t % 4, b0 + t % 4 + 4, b0 + 8 + t % 4,
                                           b0 + 8 + t % 4 + 4};
                    uint32_t v[4];
                    for (int q = 0; q < 4; ++q)
                        v[q] = (n0 < N && ks[q] < cols) ? bytes[n0 * cols + ks[q]] : 0u;
                    const uint32_t word =
                        ((v[3] & 0xFu) << 28) | ((v[2] & 0xFu) << 24) | ((v[1] & 0xFu) << 20) |
                        ((v[0] & 0xFu) << 16) | ((v[3] & 0xF0u) << 8) | ((v[2] & 0xF0u) << 4) |
                        (v[1] & 0xF0u) | ((v[0] & 0xF0u) >> 4);
                    out[((nTile * kSuper + kOuter) * 32 + t) * (inner / 2) + i / 2] = (int32_t)word;
                }
    free(bytes);
}

/*
 * Follows int4_tc_dequantize_kernel (QuantGemmKernels.cu:1170-1202), which
 * handles innerKTiles == 2 only (one word per lane): word idx -> lane, kTile,
 * nTile; n = 8*nTile + lane/4; kBase = 32*kTile + 2*(lane%4); the eight
 * nibbles at bit offsets {16,0,20,4,24,8,28,12} belong to
 * k = kBase + {1,0,9,8,17,16,25,24}.  W[n,k] = T(v-8)*scale + zero evaluated
 * with T-typed operators, i.e. each of the product and the sum is rounded to
 * T (p10/include/Half.h:183-192).  `codes_out`, when not NULL, receives the
 * raw nibble instead (used for the round-trip pin).  N must be a multiple of
 * 8 here (the packed tensor's first dimension times 8).
 */
ORC_API void orc_int4_tc_dequantize(const int32_t* packed, const void* sz, int dtype, void* W,
                                    int32_t* codes_out, int64_t N, int64_t K, int64_t group) {
    const int64_t kSuper = (K + 31) / 32;
    const int64_t total = (N / 8) * kSuper * 32;
    static const int bit[8] = {16, 0, 20, 4, 24, 8, 28, 12};
    static const int dk[8] = {1, 0, 9, 8, 17, 16, 25, 24};
    for (int64_t idx = 0; idx < total; ++idx) {
        const int lane = (int)(idx % 32);
        const int64_t kTile = (idx / 32) % kSuper;
        const int64_t nTile = idx / (32 * kSuper);
        const int64_t n = nTile * 8 + (lane >> 2);
        const int64_t kBase = kTile * 32 + 2 * (lane & 3);
        const int64_t g = (kTile * 32) / group;
        const uint32_t word = (uint32_t)packed[idx];
        for (int i = 0; i < 8; ++i) {
            const int64_t kc = kBase + dk[i];
            if (kc >= K) continue;
            const int v = (int)((word >> bit[i]) & 0xFu);
            if (codes_out) codes_out[n * K + kc] = v;
            if (W) {
                const float scale = load_as_f32(sz, dtype, (g * N + n) * 2);
                const float zero = load_as_f32(sz, dtype, (g * N + n) * 2 + 1);
                float w = round_through((float)(v - 8), dtype);
                w = round_through(w * scale, dtype);
                w = round_through(w + zero, dtype);
                store_from_f32(W, dtype, n * K + kc, w);
            }
        }
    }
}

/*
 * A7: the device op _weight_int4pack_mm (QuantGemmKernels.cu:1210-1341):
 * dequantise to a dense W[N,K] of the activation dtype (above), then
 * y = x W^T through the vendor GEMM (:1339), result in the activation dtype.
 * The vendor library's summation order is not part of the reference, so the
 * oracle accumulates in double and rounds once; `y64`, when not NULL, also
 * receives the unrounded sums.  round_w = 0 keeps W in fp32,
 * w = fmaf(code-8, scale, zero), the CPU kernel's formulation.
 * Pinned by: agreement with orc_int4_mm_cpu / torch CPU op on the same codes
 * within tolerance; _dequant_int4_reference closed form
 * (test/quantization/test_int4_modules.py:26-35).
 */
ORC_API void orc_int4_mm_tc(const void* x, int dtype, const int32_t* packed, const void* sz,
                            void* out, double* y64, int64_t M, int64_t N, int64_t K,
                            int64_t group, int round_w, int64_t row_begin, int64_t row_end) {
    float* W = (float*)malloc(sizeof(float) * (size_t)(N * K > 0 ? N * K : 1));
    if (round_w) {
        void* Wt = malloc((size_t)(N * K > 0 ? N * K : 1) * 4);
        orc_int4_tc_dequantize(packed, sz, dtype, Wt, NULL, N, K, group);
        for (int64_t i = 0; i < N * K; ++i) W[i] = load_as_f32(Wt, dtype, i);
        free(Wt);
    } else {
        int32_t* codes = (int32_t*)malloc(sizeof(int32_t) * (size_t)(N * K > 0 ? N * K : 1));
        orc_int4_tc_dequantize(packed, NULL, dtype, NULL, codes, N, K, group);
        for (int64_t n = 0; n < N; ++n)
            for (int64_t k = 0; k < K; ++k) {
                const int64_t g = k / group;
                const float scale = load_as_f32(sz, dtype, (g * N + n) * 2);
                const float zero = load_as_f32(sz, dtype, (g * N + n) * 2 + 1);
                W[n * K + k] = fmaf((float)(codes[n * K + k] - 8), scale, zero);
            }
        free(codes);
    }
    for (int64_t m = row_begin; m < row_end && m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k)
                acc += (double)load_as_f32(x, dtype, m * K + k) * (double)W[n * K + k];
            if (y64) y64[m * N + n] = acc;
            if (out) store_from_f32(out, dtype, m * N + n, (float)acc);
        }
    free(W);
}

/* ------------------------------------------------------------------------ */
/* A10: ternary 2-bit pack / unpack                                          */
/* ------------------------------------------------------------------------ */

/*
 * Follows pack_ternary (tensorplay/ao/quantization/bitnet.py:72-93): rows are
 * zero-padded to a multiple of four codes; byte = (c0&3)<<6 | (c1&3)<<4 |
 * (c2&3)<<2 | (c3&3).
 * Pinned by: the reference's literal 2x9 round trip
 * (test/quantization/test_native_1bit.py:226-234), exhaustive 3^4 byte table.
 */
ORC_API void orc_pack_ternary(const int8_t* codes, int64_t rows, int64_t cols, uint8_t* out) {
    const int64_t bytes = (cols + 3) / 4;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t b = 0; b < bytes; ++b) {
            unsigned v = 0;
            for (int q = 0; q < 4; ++q) {
                const int64_t k = b * 4 + q;
                const int c = k < cols ? codes[r * cols + k] : 0;
                v |= (unsigned)(c & 3) << (6 - 2 * q);
            }
            out[r * bytes + b] = (uint8_t)v;
        }
}

/* Follows unpack_ternary (bitnet.py:96-107): reinterpret the byte as int8 and
 * sign-extend each 2-bit field by (x << 2q) >> 6 in 8-bit arithmetic. */
ORC_API void orc_unpack_ternary(const uint8_t* packed, int64_t rows, int64_t cols, int8_t* out) {
    const int64_t bytes = (cols + 3) / 4;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t b = 0; b < bytes; ++b) {
            const int8_t x = (int8_t)packed[r * bytes + b];
            for (int q = 0; q < 4; ++q) {
                const int64_t k = b * 4 + q;
                if (k >= cols) break;
                const int8_t shifted = (int8_t)((uint8_t)x << (2 * q));
                out[r * cols + k] = (int8_t)(shifted >> 6);
            }
        }
}

/*
 * A9: follows quantize_bitnet_weight (bitnet.py:57-69) given the scale:
 * codes = clamp(round(float(W) / scale), -1, 1), round half to even.  The
 * scale itself (mean |W| clamped to eps, bitnet.py:48-54) is a tensor-library
 * reduction whose summation order the reference does not fix; callers
 * compute it (in double) and pass the fp32 value in.
 * Pinned by: the literal 2x4 weight and codes in
 * test/quantization/test_native_1bit.py:213-224.
 */
ORC_API void orc_quantize_bitnet_weight(const float* w, int64_t numel, float scale, int8_t* codes) {
    for (int64_t i = 0; i < numel; ++i) {
        float q = nearbyintf(w[i] / scale);
        q = q < -1.0f ? -1.0f : (q > 1.0f ? 1.0f : q);
        codes[i] = (int8_t)q;
    }
}

/* ------------------------------------------------------------------------ */
/* A12: PackedWeight prepack + linear run (float output)                     */
/* ------------------------------------------------------------------------ */

/*
 * Follows _quantized_weight_prepack_cpu (p10/src/backend/cpu/QuantPacked.cpp
 * :519-533; shape rule p10/include/QuantPacked.h:51-56): rows copied into a
 * zero-filled [N, ceil(K/32)*32] int8 matrix, offsets[n] = sum_k w[n,k].
 */
ORC_API void orc_weight_prepack(const int8_t* w, int64_t N, int64_t K, int8_t* packed,
                                int64_t* offsets) {
    const int64_t padded = (K + 31) / 32 * 32;
    memset(packed, 0, (size_t)(N * padded));
    for (int64_t n = 0; n < N; ++n) {
        if (K) memcpy(packed + n * padded, w + n * K, (size_t)K);
        int64_t sum = 0;
        for (int64_t k = 0; k < K; ++k) sum += w[n * K + k];
        offsets[n] = sum;
    }
}

/*
 * Follows the linear, output_float branch of run<X> (QuantPacked.cpp:420-516)
 * with packed_real_value (p10/include/QuantPacked.h:133-139):
 *   acc   = dot(x, w) - xz*offsets[n] - wz[n]*sum(x) + K*xz*wz[n]
 *   value = fmaf(float(acc), float(xs) * ws[n], bias[n] or 0)
 * The hot path calls it with xs = 1, xz = 0, ws = 1, wz = 0 and no bias
 * (bitnet.py:234-237, int8_mixed_precision.py:72-76), i.e. float(dot).
 * Pinned by: the int64 closed form of
 * test/quantization/test_packed_quantization.py:54-58.
 */
ORC_API void orc_packed_run_linear_float(const void* x, int x_unsigned, double xs, int64_t xz,
                                         const int8_t* packed, const int64_t* offsets,
                                         const float* ws, const int64_t* wz, const float* bias,
                                         float* out, int64_t rows, int64_t N, int64_t K) {
    const int64_t padded = (K + 31) / 32 * 32;
    for (int64_t r = 0; r < rows; ++r) {
        int64_t row_sum = 0;
        for (int64_t k = 0; k < K; ++k)
            row_sum += x_unsigned ? (int64_t)((const uint8_t*)x)[r * K + k]
                                  : (int64_t)((const int8_t*)x)[r * K + k];
        for (int64_t n = 0; n < N; ++n) {
            int64_t raw = 0;
            for (int64_t k = 0; k < K; ++k) {
                const int64_t xv = x_unsigned ? (int64_t)((const uint8_t*)x)[r * K + k]
                                              : (int64_t)((const int8_t*)x)[r * K + k];
                raw += xv * packed[n * padded + k];
            }
            const int64_t acc = raw - xz * offsets[n] - wz[n] * row_sum + K * xz * wz[n];
            out[r * N + n] = fmaf((float)acc, (float)xs * ws[n], bias ? bias[n] : 0.0f);
        }
    }
}

/* ------------------------------------------------------------------------ */
/* A11: BitNet packed linear                                                 */
/* ------------------------------------------------------------------------ */

/*
 * Follows bitnet_linear_packed (bitnet.py:215-241) after the activation
 * quantizer: acc[m,n] = sum_k x_i8[m,k] * code[n,k] (exact int32), and
 * y = (float(acc) * row_scale[m]) * w_scale (+ bias[n]), fp32 multiplies in
 * the reference's left-to-right order (`out * row_scale * scale`, :238).
 * `acc_out` (optional) receives the integer sums, `out` the fp32 result
 * rounded once to out_dtype.
 * Pinned by: manual_bitnet_linear closed form
 * (test/quantization/test_native_1bit.py:200-210).
 */
ORC_API void orc_ternary_mm(const int8_t* x, const float* row_scale, const uint8_t* packed,
                            float w_scale, const float* bias, int64_t M, int64_t N, int64_t K,
                            void* out, int out_dtype, int32_t* acc_out) {
    const int64_t bytes = (K + 3) / 4;
    int8_t* codes = (int8_t*)malloc((size_t)(N * K > 0 ? N * K : 1));
    orc_unpack_ternary(packed, N, K, codes);
    (void)bytes;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            int32_t acc = 0;
            for (int64_t k = 0; k < K; ++k) acc += (int32_t)x[m * K + k] * (int32_t)codes[n * K + k];
            if (acc_out) acc_out[m * N + n] = acc;
            if (out) {
                float v = (float)acc * row_scale[m];
                v = v * w_scale;
                if (bias) v = v + bias[n];
                store_from_f32(out, out_dtype, m * N + n, v);
            }
        }
    free(codes);
}

/* ---- _weight_int8pack_mm ------------------------------------------------------------------------
 * out[m,n] = cast((sum_k float(x[m,k]) * float(w[n,k])) * scale[n]); x is converted to fp32 first and
 * the sum is an fp32 fma chain (p10/src/backend/cuda/QuantGemmKernels.cu:86-130, 339-405; the device
 * kernel strides k over lanes, so its summation order differs - tolerance, not bit parity).
 * y64 (optional) receives the same sums evaluated in double precision.
 * Pinned by: the literal 2x4 / 3x4 example and closed form (x @ w.T) * s of
 * test/test_mps.py:1052-1061, and the float64 product.
 */
ORC_API void orc_weight_int8pack_mm(const void* x, int dtype, const int8_t* w, const float* scale,
                                    int64_t M, int64_t N, int64_t K, void* out, double* y64) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float acc = 0.0f;
            double acc64 = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                const float xv = load_as_f32(x, dtype, m * K + k);
                acc = fmaf((float)w[n * K + k], xv, acc);
                acc64 += (double)w[n * K + k] * (double)xv;
            }
            store_from_f32(out, dtype, m * N + n, acc * scale[n]);
            if (y64) y64[m * N + n] = acc64 * (double)scale[n];
        }
}

/* ------------------------------------------------------------------------ */
/* rms_norm                                                                   */
/* ------------------------------------------------------------------------ */

/* rms_norm over the last dimension, rows of K: the CPU kernel of the reference
 * (p10/src/backend/cpu/NormalizationKernels.cpp:1355-1453).  float32 rows
 * (:1389-1396) and float16 / bfloat16 rows (:1424-1449) follow the same steps in
 * float: acc += v * v serially, inv = 1 / sqrt(acc / K + eps), v = x * inv,
 * v *= w, one rounding to the storage type.  weight may be NULL.  y64, when not
 * NULL, receives the same formula evaluated in double on the same inputs (the
 * composite of tensorplay/nn/functional.py:2350-2372 without its roundings).
 * Pinned by: torch.nn.functional.rms_norm on the CPU (a library twin: float32
 * within 2 ulp, 16-bit types within one rounding), the float64 closed form,
 * exact invariance under scaling the row by a power of two at eps = 0, a
 * constant row (x = c: out = sign(c) w up to rounding), zero rows (out = 0).
 */
ORC_API void orc_rms_norm(const void* x, int dtype, int64_t M, int64_t K, const void* weight, float eps,
                          void* out, double* y64) {
    for (int64_t m = 0; m < M; ++m) {
        float acc = 0.0f;
        double acc64 = 0.0;
        for (int64_t k = 0; k < K; ++k) {
            const float v = load_as_f32(x, dtype, m * K + k);
            acc += v * v;
            acc64 += (double)v * (double)v;
        }
        const float inv = 1.0f / sqrtf(acc / (float)K + eps);
        const double inv64 = 1.0 / sqrt(acc64 / (double)K + (double)eps);
        for (int64_t k = 0; k < K; ++k) {
            const float xv = load_as_f32(x, dtype, m * K + k);
            float v = xv * inv;
            const float w = weight ? load_as_f32(weight, dtype, k) : 1.0f;
            if (weight) v *= w;
            store_from_f32(out, dtype, m * K + k, v);
            if (y64) y64[m * K + k] = (double)xv * inv64 * (double)w;
        }
    }
}

/* ------------------------------------------------------------------------ */
/* Block-wise affine quantizer                                               */
/* ------------------------------------------------------------------------ */

/* Block of a row-major linear index in the grid of ceil(size / block) blocks
 * (AffineGroupParams::block_of and make_affine_group_params,
 * p10/src/backend/cpu/QuantKernels.cpp:316-360). */
static int64_t affine_block_of(int64_t linear, int ndim, const int64_t* sizes, const int64_t* block_size) {
    int64_t b = 0, size_stride = 1, block_stride = 1;
    for (int d = ndim - 1; d >= 0; --d) {
        int64_t blk = block_size[d] < sizes[d] ? block_size[d] : sizes[d];
        if (blk <= 0) blk = 1;
        const int64_t per_dim = (sizes[d] + blk - 1) / blk;
        const int64_t coord = (linear / size_stride) % sizes[d];
        b += (coord / blk) * block_stride;
        size_stride *= sizes[d];
        block_stride *= per_dim;
    }
    return b;
}

/* bits per element of a storage tag (0 int8, 1 uint8, 2 int32, 3 4-bit, 4 2-bit, 5 1-bit) */
static int affine_bits(int storage) {
    static const int bits[6] = {8, 8, 32, 4, 2, 1};
    return bits[storage];
}

/*
 * quantize_affine on float32 input.  One scale / zero point per block, or a
 * single one for all blocks (n_scales / n_zeros == 1); n_zeros == 0: none.
 * Byte and int32 storages: quantize_affine_kernel, QuantKernels.cpp:365-388
 * (double position, clamp on the int64).  Packed storages:
 * quantize_affine_subbyte_kernel, :406-438 (float position, int64 cut to its
 * low 32 bits, clamp on the int32, low bits first).  The 2-D group kernels
 * (:457-478, :504-537) and the device kernels (AffineQuantKernels.cu:818-884)
 * compute the same values.
 *
 * Pinned by: torch.quantize_per_tensor / quantize_per_channel int_repr on the
 * CPU (library twins for one block and for per-row blocks), the numpy closed
 * form clamp(rint(x * (1/s)) + z) for grouped and tiled grids, the
 * least-significant-first packing formula of
 * test/quantization/test_native_1bit.py:43-50, and hand-computed edge cases
 * (NaN, +-inf, 2^40, zero scale).
 */
ORC_API void orc_quantize_affine(const float* x, int ndim, const int64_t* sizes, const int64_t* block_size,
                                 const float* scales, int64_t n_scales, const float* zeros, int64_t n_zeros,
                                 int storage, int64_t qmin, int64_t qmax, void* out) {
    int64_t numel = 1;
    for (int d = 0; d < ndim; ++d) numel *= sizes[d];
    const int bits = affine_bits(storage);
    if (bits < 8) memset(out, 0, (size_t)((numel * bits + 7) / 8));
    for (int64_t i = 0; i < numel; ++i) {
        const int64_t b = affine_block_of(i, ndim, sizes, block_size);
        const float s = scales[n_scales == 1 ? 0 : b];
        const float inv = s == 0.f ? 1.f : 1.f / s;
        const float rounded = nearbyintf(x[i] * inv);
        const float position = n_zeros ? rounded + zeros[n_zeros == 1 ? 0 : b] : rounded;
        const int64_t wide = (position >= -0x1p63f && position < 0x1p63f) ? (int64_t)position : INT64_MIN;
        if (bits >= 8) {
            int64_t q = wide < qmin ? qmin : wide > qmax ? qmax : wide;
            if (storage == 0) ((int8_t*)out)[i] = (int8_t)q;
            else if (storage == 1) ((uint8_t*)out)[i] = (uint8_t)q;
            else ((int32_t*)out)[i] = (int32_t)q;
        } else {
            const int pack = 8 / bits;
            int32_t q = (int32_t)(uint32_t)wide;
            q = q < (int32_t)qmin ? (int32_t)qmin : q > (int32_t)qmax ? (int32_t)qmax : q;
            ((uint8_t*)out)[i / pack] |= (uint8_t)((uint8_t)q << ((i % pack) * bits));
        }
    }
}

/*
 * dequantize_affine: (float(code) - zero) * scale, QuantKernels.cpp:391-404
 * (bytes, int32) and :440-455 (packed storages).
 * Pinned by: the closed form in numpy float32, round trips of
 * orc_quantize_affine codes, torch dequantize() of per-tensor / per-channel
 * quantized CPU tensors.
 */
ORC_API void orc_dequantize_affine(const void* codes, int storage, int ndim, const int64_t* sizes,
                                   const int64_t* block_size, const float* scales, int64_t n_scales,
                                   const float* zeros, int64_t n_zeros, float* out) {
    int64_t numel = 1;
    for (int d = 0; d < ndim; ++d) numel *= sizes[d];
    const int bits = affine_bits(storage);
    for (int64_t i = 0; i < numel; ++i) {
        const int64_t b = affine_block_of(i, ndim, sizes, block_size);
        float code;
        if (storage == 0) code = (float)((const int8_t*)codes)[i];
        else if (storage == 1) code = (float)((const uint8_t*)codes)[i];
        else if (storage == 2) code = (float)((const int32_t*)codes)[i];
        else {
            const int pack = 8 / bits;
            code = (float)((((const uint8_t*)codes)[i / pack] >> ((i % pack) * bits)) & ((1 << bits) - 1));
        }
        out[i] = (code - (n_zeros ? zeros[n_zeros == 1 ? 0 : b] : 0.f)) * scales[n_scales == 1 ? 0 : b];
    }
}

/* ------------------------------------------------------------------------ */
/* Packed n-bit weight-only linear (int2 / intx / binary modules)            */
/* ------------------------------------------------------------------------ */

/* shift of code i (0 .. 8/bits - 1) inside its byte: first code in the most
 * significant bits (pack_intx, tensorplay/ao/quantization/intx_weight_only.py:55-58;
 * pack_int2, int2_weight_only.py:82-87) or, lsb_first, code i in bit i * bits
 * (pack_binary, binary.py:66-70). */
static int lowbit_shift(int i, int bits, int lsb_first) { return lsb_first ? i * bits : 8 - (i + 1) * bits; }

/*
 * codes uint8 [rows, cols] -> packed uint8 [rows, ceil(cols / (8 / bits))], tail padded with zeros.
 * Pinned by: a numpy restatement of the reference's strided-slice formulas, the shapes of
 * test/quantization/test_int2_binary_modules.py:57-66, 129-137 and pack/unpack round trips.
 */
ORC_API void orc_lowbit_pack(const uint8_t* codes, int bits, int lsb_first, int64_t rows, int64_t cols, uint8_t* packed) {
    const int per_byte = 8 / bits;
    const int64_t pitch = (cols + per_byte - 1) / per_byte;
    memset(packed, 0, (size_t)(rows * pitch));
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c)
            packed[r * pitch + c / per_byte] |=
                (uint8_t)((codes[r * cols + c] & ((1 << bits) - 1)) << lowbit_shift((int)(c % per_byte), bits, lsb_first));
}

/* unpack_intx (intx_weight_only.py:62-80) / unpack_int2 (int2_weight_only.py:91-103) / unpack_binary (binary.py:74-85) */
ORC_API void orc_lowbit_unpack(const uint8_t* packed, int bits, int lsb_first, int64_t rows, int64_t cols, uint8_t* codes) {
    const int per_byte = 8 / bits;
    const int64_t pitch = (cols + per_byte - 1) / per_byte;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c)
            codes[r * cols + c] =
                (uint8_t)((packed[r * pitch + c / per_byte] >> lowbit_shift((int)(c % per_byte), bits, lsb_first)) & ((1 << bits) - 1));
}

/*
 * _intx_mm / _int2_mm (intx_weight_only.py:110-133, int2_weight_only.py:115-139): the dense weight
 * dq[n,k] = (float(code) - zero[g,n]) * scale[g,n] in float32, then out = x @ dq.T (+ bias).
 * sz: float32 [K / group][N][2].  `dense` (optional) receives dq; `out` is rounded to `dtype` from a
 * float32 fma chain over k; `y64` (optional) is the same sum in double from the float32 dq.
 * _binary_mm (binary.py:88-95) is the case bits = 1, lsb_first, one group, scale' = 2 scale, zero = 0.5:
 * (bit - 0.5) * 2 s = (2 bit - 1) * s exactly.
 * Pinned by: numpy float64 x @ dq.T with dq from the closed form on independently unpacked codes; the
 * reference test's own check (test_int2_binary_modules.py:69-89, 140-155) restated in numpy; at 8 bits the
 * reference's unpack -> int8 -> float chain written out in numpy on bytes of 128 and more.
 */
ORC_API void orc_lowbit_mm(const void* x, int dtype, const uint8_t* packed, int bits, int lsb_first, const float* sz,
                           const float* bias, int64_t M, int64_t N, int64_t K, int64_t group, void* out, double* y64,
                           float* dense) {
    const int per_byte = 8 / bits;
    const int64_t pitch = (K + per_byte - 1) / per_byte;
    for (int64_t n = 0; n < N; ++n) {
        for (int64_t m = 0; m < (M > 0 ? M : 1); ++m) {
            float acc = 0.0f;
            double acc64 = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                const int code = (packed[n * pitch + k / per_byte] >> lowbit_shift((int)(k % per_byte), bits, lsb_first)) & ((1 << bits) - 1);
                const float* p = sz + ((k / group) * N + n) * 2;
                /* unpack_intx ends in codes.to(int8) (intx_weight_only.py:80) and _dequantize_intx converts that int8
                 * to float (:119): at 8 bits a byte of 128 or more counts as byte - 256 */
                const float dq = ((float)(bits == 8 ? (int)(int8_t)code : code) - p[1]) * p[0];
                if (dense && m == 0) dense[n * K + k] = dq;
                if (M > 0) {
                    const float xv = load_as_f32(x, dtype, m * K + k);
                    acc = fmaf(dq, xv, acc);
                    acc64 += (double)dq * (double)xv;
                }
            }
            if (M > 0) {
                if (bias) { acc += bias[n]; acc64 += (double)bias[n]; }
                if (out) store_from_f32(out, dtype, m * N + n, acc);
                if (y64) y64[m * N + n] = acc64;
            }
        }
    }
}
