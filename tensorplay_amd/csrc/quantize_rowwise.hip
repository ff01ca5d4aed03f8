// Fused row-wise signed quantizer for gfx950.
//
// One 256-thread workgroup per row (rows of up to 1024 elements: a lane group of 8..64 lanes per
// row, several rows per workgroup).  The row is read from HBM once, kept in
// registers (8 elements per 16/32-byte vector load, up to 8 such chunks per
// lane), reduced to its absolute maximum with a 64-lane butterfly and one LDS
// exchange between the four wavefronts, and written back as int8 codes with
// 8-byte stores (rows of more than 16384 elements: 1024 threads).  Rows longer than the register budget
// (K > 65536) or rows
// that cannot be vector-loaded (K % 8 != 0) take the streaming kernel, which
// reads the row a second time (the second read comes from L2).
//
// Arithmetic (bit-exact with the reference's CPU kernel,
// p10/include/QuantNativeImpl.h:1162-1187 and
// p10/src/backend/cpu/LowBitGemmKernels.cpp:19-52):
//   absmax = max |float(x)|;  scale = fmaxf(absmax, eps) / divisor  (IEEE divide)
//   code   = clamp(rintf(float(x) / scale), qmin, qmax)              (IEEE divide, RNE)
#include "tpq_common.h"

namespace tpq {
namespace {

constexpr int kThreads = 256;
constexpr int kVec = 8;  // elements per lane per chunk
// Rows up to this length: one wavefront (or a part of one) per row.  Longer rows on one wavefront were measured
// (2048 x 4096 bfloat16: 7.0 us against 6.6 with four wavefronts per row, 8.9 against 7.1 from HBM; two wavefronts per
// row: 8.3 against 7.9): a quarter of the wavefronts to launch, but too few loads in flight per compute unit.
constexpr int kSubwaveMaxK = 1024;

// -DTPQ_QUANT_STAMPS (a measuring build of its own, never the shipped library): every workgroup of the register-cached
// kernel leaves six readings of the shader clock (entry, loads issued, own data arrived and reduced, row maximum known,
// stores issued, stores acknowledged: the counters of different compute units do not share a zero, so only differences
// inside a workgroup mean something) and two of the chip-wide 100 MHz clock (entry, end).
#ifdef TPQ_QUANT_STAMPS
constexpr int kStampSlots = 8, kStampRows = 8192;
__device__ unsigned long long g_quant_stamps[kStampRows * kStampSlots];
#define TPQ_QUANT_STAMP(I)                                                                                              \
    do {                                                                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        if (threadIdx.x == 0 && blockIdx.x < kStampRows) g_quant_stamps[blockIdx.x * kStampSlots + (I)] = __builtin_amdgcn_s_memtime(); \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
    } while (0)
#else
#define TPQ_QUANT_STAMP(I) do { } while (0)
#endif

struct QParams {
    float eps, divisor;
    int qmin, qmax, sign_mode;
    int no_clamp;  // no quotient |v| / scale, |v| <= absmax, can round outside [qmin, qmax]
};

__device__ __forceinline__ int quantize_one(float v, float scale, const QParams& p) {
    if (p.sign_mode) return v >= 0.0f ? p.qmax : p.qmin;
    // __fdiv_rn: correctly rounded division regardless of compiler flags
    float q = rintf(__fdiv_rn(v, scale));
    q = fminf(fmaxf(q, static_cast<float>(p.qmin)), static_cast<float>(p.qmax));
    return static_cast<int>(q);
}

// Eight codes with one reciprocal instead of eight divisions, same bits as quantize_one.
// q = v * (1/scale) is within 2^-21 relative of the true quotient, |quotient| <= 128 here, so its
// absolute error is below 2^-14.  If q lies at least 2^-13 inside (c - 1/2, c + 1/2), so does the
// correctly rounded quotient, and both round to c.  Otherwise (about one element in a few thousand;
// also NaN and infinities) the element is redone with the IEEE division.
// The codes leave as two packed words.  v_cvt_pk_u8_f32 converts a float to an unsigned byte (saturating at 0 and
// 255) and drops it into one byte of a register: the rounded quotient c is an integer already, so c + 128 converts
// exactly, the upper clamp is the saturation when qmax = 127, and one xor takes the 128 off the four bytes again.
// Four instructions per code less than clamp, convert, mask, shift, or.
__device__ __forceinline__ void quantize_eight_packed(const float (&v)[kVec], float scale, float inv_scale, const QParams& p,
                                                      uint32_t& lo, uint32_t& hi) {
    bool redo = false;
    uint32_t word[2] = {0u, 0u};
    const float qmin = static_cast<float>(p.qmin), qmax = static_cast<float>(p.qmax);
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
        const float q = v[i] * inv_scale;
        const float c = rintf(q);
        redo |= !(fabsf(q - c) <= 0.5f - 0x1p-13f);
        const float biased = fminf(fmaxf(c, qmin), qmax) + 128.0f;  // 0 .. 255, an integer
        word[i >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(biased, i & 3, word[i >> 2]);
    }
    lo = word[0] ^ 0x80808080u;
    hi = word[1] ^ 0x80808080u;
    // Rare (one element in a few thousand).  Behind a branch the whole wavefront takes or skips, with a statement the
    // compiler may not move: left as a plain "if", the eight divisions were computed for every chunk and selected away.
    // Rare (one element in a few thousand).  Behind a branch the whole wavefront takes or skips, and with the divisor
    // passed through a statement the compiler may not move: as a plain "if", the eight divisions were hoisted above the
    // branch, computed for every chunk and selected away.
    if (__builtin_amdgcn_ballot_w64(redo) != 0) {
        float divisor = scale;
        asm volatile("; elements redone with the division" : "+v"(divisor));
        if (redo) {
            lo = hi = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                lo |= (static_cast<uint32_t>(quantize_one(v[i], divisor, p)) & 0xFFu) << (8 * i);
                hi |= (static_cast<uint32_t>(quantize_one(v[i + 4], divisor, p)) & 0xFFu) << (8 * i);
            }
        }
    }
}

// The same codes with fewer instructions, for parameters under which no quotient can leave the code range
// (rint(divisor (1 + 2^-20)) <= qmax and >= -qmin, true for the usual divisor = qmax = -qmin = 127): no clamp is
// needed, and the code is read off the mantissa.  t = fma(v, 1/scale, 1.5 * 2^23) rounds the exact product to the
// nearest integer (ties to even) and leaves it in two's complement in the low mantissa bits; c = t - 1.5 * 2^23 is that
// integer, r = fma(v, 1/scale, -c) its distance from the product.  The product is within 2^-16 of the correctly rounded
// quotient the reference rounds, so |r| <= 1/2 - 2^-13 proves both round to c; anything else (also NaN) is redone with
// the division.  Five instructions per code and three byte permutes per four codes.
__device__ __forceinline__ void quantize_eight_lean(const float (&v)[kVec], float scale, float inv_scale, const QParams& p,
                                                    uint32_t& lo, uint32_t& hi) {
    constexpr float kMagic = 12582912.0f;  // 1.5 * 2^23
    bool redo = false;
    uint32_t t[kVec];
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
        const float tf = __builtin_fmaf(v[i], inv_scale, kMagic);
        const float c = tf - kMagic;
        const float r = __builtin_fmaf(v[i], inv_scale, -c);
        redo |= !(fabsf(r) <= 0.5f - 0x1p-13f);
        t[i] = __builtin_bit_cast(uint32_t, tf);
    }
    // v_perm_b32(a, b, sel): selector bytes 0..3 take bytes of b, 4..7 of a, 0x0c a zero byte
    lo = __builtin_amdgcn_perm(t[1], t[0], 0x0c0c0400u) | __builtin_amdgcn_perm(t[3], t[2], 0x04000c0cu);
    hi = __builtin_amdgcn_perm(t[5], t[4], 0x0c0c0400u) | __builtin_amdgcn_perm(t[7], t[6], 0x04000c0cu);
    // Rare (one element in a few thousand).  Behind a branch the whole wavefront takes or skips, with a statement the
    // compiler may not move: left as a plain "if", the eight divisions were computed for every chunk and selected away.
    // Rare (one element in a few thousand).  Behind a branch the whole wavefront takes or skips, and with the divisor
    // passed through a statement the compiler may not move: as a plain "if", the eight divisions were hoisted above the
    // branch, computed for every chunk and selected away.
    if (__builtin_amdgcn_ballot_w64(redo) != 0) {
        float divisor = scale;
        asm volatile("; elements redone with the division" : "+v"(divisor));
        if (redo) {
            lo = hi = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                lo |= (static_cast<uint32_t>(quantize_one(v[i], divisor, p)) & 0xFFu) << (8 * i);
                hi |= (static_cast<uint32_t>(quantize_one(v[i + 4], divisor, p)) & 0xFFu) << (8 * i);
            }
        }
    }
}

// Block-wide max over THREADS threads; every thread gets the result.
template <int THREADS = kThreads>
__device__ __forceinline__ float block_max(float v, float* smem) {
    v = wave_max(v);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float r = smem[0];
#pragma unroll
    for (int w = 1; w < THREADS / kWave; ++w) r = fmaxf(r, smem[w]);
    return r;
}

template <int DT>
__device__ __forceinline__ void load_chunk(const typename Elem<DT>::storage* p, float (&v)[kVec]) {
    if constexpr (DT == TPQ_DTYPE_F32) {
        const uint4 a = nt_load(reinterpret_cast<const uint4*>(p)), b = nt_load(reinterpret_cast<const uint4*>(p) + 1);
        v[0] = __builtin_bit_cast(float, a.x); v[1] = __builtin_bit_cast(float, a.y);
        v[2] = __builtin_bit_cast(float, a.z); v[3] = __builtin_bit_cast(float, a.w);
        v[4] = __builtin_bit_cast(float, b.x); v[5] = __builtin_bit_cast(float, b.y);
        v[6] = __builtin_bit_cast(float, b.z); v[7] = __builtin_bit_cast(float, b.w);
    } else {
        const uint4 raw = nt_load(reinterpret_cast<const uint4*>(p));
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = Elem<DT>::load(static_cast<uint16_t>(w[i] & 0xFFFFu));
            v[2 * i + 1] = Elem<DT>::load(static_cast<uint16_t>(w[i] >> 16));
        }
    }
}

// Row cached in registers: CHUNKS * THREADS * 8 >= K, K % 8 == 0.
template <int DT, int CHUNKS, int THREADS = kThreads>
__global__ __launch_bounds__(THREADS) void quantize_rows_cached(
    const typename Elem<DT>::storage* __restrict__ x, int8_t* __restrict__ codes,
    float* __restrict__ scales, int K, QParams p) {
    __shared__ float smem[THREADS / kWave];
    const int64_t row = blockIdx.x;
    const auto* xr = x + row * K;
    int8_t* cr = codes + row * K;

#ifdef TPQ_QUANT_STAMPS
    if (threadIdx.x == 0 && blockIdx.x < kStampRows) g_quant_stamps[blockIdx.x * kStampSlots + 6] = __builtin_amdgcn_s_memrealtime();
#endif
    TPQ_QUANT_STAMP(0);
    float v[CHUNKS][kVec];
    float absmax = 0.0f;
    // No branch around the loads: at the join of a branch the compiler waits for every outstanding load, which made
    // the chunks one round trip to memory each.  A chunk past the end re-reads the last chunk of the row: the same
    // elements again do not change the maximum, and nothing is stored for it.
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k0 = (c * THREADS + threadIdx.x) * kVec;
        load_chunk<DT>(xr + (k0 < K ? k0 : K - kVec), v[c]);
    }
    TPQ_QUANT_STAMP(1);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
        for (int i = 0; i < kVec; ++i) absmax = fmaxf(absmax, fabsf(v[c][i]));
    absmax = wave_max(absmax);
    TPQ_QUANT_STAMP(2);
    absmax = block_max<THREADS>(absmax, smem);
    TPQ_QUANT_STAMP(3);
    const float scale = __fdiv_rn(fmaxf(absmax, p.eps), p.divisor);
    if (threadIdx.x == 0) scales[row] = scale;
    // the shortcut needs |quotient| <= 128 and a finite reciprocal: true for every scale the formula
    // above produces from finite inputs with divisor <= 128; anything else takes the divisions
    const float inv_scale = __fdiv_rn(1.0f, scale);
    const bool shortcut = !p.sign_mode && p.divisor <= 128.0f && inv_scale < 3.0e38f && absmax <= 3.0e38f;
    const bool lean = shortcut && p.no_clamp;

#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k0 = (c * THREADS + threadIdx.x) * kVec;
        if (k0 < K) {
            uint32_t lo = 0, hi = 0;
            if (lean) {
                quantize_eight_lean(v[c], scale, inv_scale, p, lo, hi);
            } else if (shortcut) {
                quantize_eight_packed(v[c], scale, inv_scale, p, lo, hi);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    lo |= (static_cast<uint32_t>(quantize_one(v[c][i], scale, p)) & 0xFFu) << (8 * i);
                    hi |= (static_cast<uint32_t>(quantize_one(v[c][i + 4], scale, p)) & 0xFFu) << (8 * i);
                }
            }
            *reinterpret_cast<uint2*>(cr + k0) = make_uint2(lo, hi);
        }
    }
#ifdef TPQ_QUANT_STAMPS
    TPQ_QUANT_STAMP(4);
    __builtin_amdgcn_s_waitcnt(0);  // every store of this wavefront acknowledged
    TPQ_QUANT_STAMP(5);
    if (threadIdx.x == 0 && blockIdx.x < kStampRows) g_quant_stamps[blockIdx.x * kStampSlots + 7] = __builtin_amdgcn_s_memrealtime();
#endif
}

// Short rows (K <= LANES * CHUNKS * 8, K % 8 == 0): LANES lanes of a wavefront per row, so a workgroup
// takes 256 / LANES rows and no lane idles; the maximum is a butterfly inside the lane group, no LDS.
template <int DT, int LANES, int CHUNKS>
__global__ __launch_bounds__(kThreads) void quantize_rows_subwave(
    const typename Elem<DT>::storage* __restrict__ x, int8_t* __restrict__ codes,
    float* __restrict__ scales, int64_t M, int K, QParams p) {
    constexpr int kRows = kThreads / LANES;
    const int sub = threadIdx.x % LANES;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kRows + threadIdx.x / LANES;
    const bool live = row < M;  // dead lanes still take part in the butterfly
    const auto* xr = x + (live ? row : 0) * K;
    int8_t* cr = codes + (live ? row : 0) * K;

    float v[CHUNKS][kVec];
    float absmax = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k0 = (c * LANES + sub) * kVec;
        load_chunk<DT>(xr + (k0 < K ? k0 : K - kVec), v[c]);  // branch-free: see quantize_rows_cached; dead rows read row 0
    }
    if (live) {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
            for (int i = 0; i < kVec; ++i) absmax = fmaxf(absmax, fabsf(v[c][i]));
    }
#pragma unroll
    for (int off = LANES / 2; off >= 1; off >>= 1) absmax = fmaxf(absmax, __shfl_xor(absmax, off));
    const float scale = __fdiv_rn(fmaxf(absmax, p.eps), p.divisor);
    if (live && sub == 0) scales[row] = scale;
    const float inv_scale = __fdiv_rn(1.0f, scale);
    const bool shortcut = !p.sign_mode && p.divisor <= 128.0f && inv_scale < 3.0e38f && absmax <= 3.0e38f;  // as above
    const bool lean = shortcut && p.no_clamp;

#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k0 = (c * LANES + sub) * kVec;
        if (live && k0 < K) {
            uint32_t lo = 0, hi = 0;
            if (lean) {
                quantize_eight_lean(v[c], scale, inv_scale, p, lo, hi);
            } else if (shortcut) {
                quantize_eight_packed(v[c], scale, inv_scale, p, lo, hi);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    lo |= (static_cast<uint32_t>(quantize_one(v[c][i], scale, p)) & 0xFFu) << (8 * i);
                    hi |= (static_cast<uint32_t>(quantize_one(v[c][i + 4], scale, p)) & 0xFFu) << (8 * i);
                }
            }
            *reinterpret_cast<uint2*>(cr + k0) = make_uint2(lo, hi);
        }
    }
}

// Any K: two passes over the row with scalar accesses.
template <int DT>
__global__ __launch_bounds__(kThreads) void quantize_rows_streaming(
    const typename Elem<DT>::storage* __restrict__ x, int8_t* __restrict__ codes,
    float* __restrict__ scales, int64_t K, QParams p) {
    __shared__ float smem[kThreads / kWave];
    const int64_t row = blockIdx.x;
    const auto* xr = x + row * K;
    int8_t* cr = codes + row * K;
    float absmax = 0.0f;
    for (int64_t k = threadIdx.x; k < K; k += kThreads) absmax = fmaxf(absmax, fabsf(Elem<DT>::load(xr[k])));
    absmax = block_max(absmax, smem);
    const float scale = __fdiv_rn(fmaxf(absmax, p.eps), p.divisor);
    if (threadIdx.x == 0) scales[row] = scale;
    for (int64_t k = threadIdx.x; k < K; k += kThreads)
        cr[k] = static_cast<int8_t>(quantize_one(Elem<DT>::load(xr[k]), scale, p));
}

template <int DT>
int launch(const void* x, int64_t M, int64_t K, const QParams& p, int8_t* codes, float* scales,
           hipStream_t stream) {
    using S = typename Elem<DT>::storage;
    const S* xp = static_cast<const S*>(x);
    const dim3 grid(static_cast<unsigned>(M)), block(kThreads);
    const bool vec_ok = (K % kVec == 0) && aligned(x, 16) && aligned(codes, 8) && K <= 8 * 1024 * kVec;
    if (vec_ok && K <= kSubwaveMaxK) {
        const int k = static_cast<int>(K);
        auto run = [&](auto lanes, auto chunks) {
            constexpr int L = decltype(lanes)::value, C = decltype(chunks)::value;
            const dim3 g(static_cast<unsigned>((M + kThreads / L - 1) / (kThreads / L)));
            quantize_rows_subwave<DT, L, C><<<g, block, 0, stream>>>(xp, codes, scales, M, k, p);
        };
        using std::integral_constant;
        if (K <= 64) run(integral_constant<int, 8>{}, integral_constant<int, 1>{});
        else if (K <= 128) run(integral_constant<int, 16>{}, integral_constant<int, 1>{});
        else if (K <= 256) run(integral_constant<int, 32>{}, integral_constant<int, 1>{});
        else if (K <= 512) run(integral_constant<int, 64>{}, integral_constant<int, 1>{});
        else run(integral_constant<int, 64>{}, integral_constant<int, 2>{});
    } else if (vec_ok) {
        const int chunks = static_cast<int>((K + kThreads * kVec - 1) / (kThreads * kVec));
        const int k = static_cast<int>(K);
        if (chunks <= 1) quantize_rows_cached<DT, 1><<<grid, block, 0, stream>>>(xp, codes, scales, k, p);
        else if (chunks <= 2) quantize_rows_cached<DT, 2><<<grid, block, 0, stream>>>(xp, codes, scales, k, p);
        else if (chunks <= 4) quantize_rows_cached<DT, 4><<<grid, block, 0, stream>>>(xp, codes, scales, k, p);
        else if (chunks <= 8) quantize_rows_cached<DT, 8><<<grid, block, 0, stream>>>(xp, codes, scales, k, p);
        else if (chunks <= 16) quantize_rows_cached<DT, 4, 1024><<<grid, 1024, 0, stream>>>(xp, codes, scales, k, p);
        else quantize_rows_cached<DT, 8, 1024><<<grid, 1024, 0, stream>>>(xp, codes, scales, k, p);
    } else {
        quantize_rows_streaming<DT><<<grid, block, 0, stream>>>(xp, codes, scales, K, p);
    }
    return check_launch("tpq_quantize_rowwise");
}

}  // namespace
}  // namespace tpq

#ifdef TPQ_QUANT_STAMPS
// [rows][8] clock readings of the last launch of the register-cached kernel (rows beyond 8192 are not recorded)
TPQ_EXPORT int tpq_quantize_stamps_read(unsigned long long* host, int64_t rows) {
    using namespace tpq;
    TPQ_REQUIRE(host && rows >= 0 && rows <= kStampRows, TPQ_ERR_INVALID_VALUE, "quantize stamps: at most %d rows", kStampRows);
    const hipError_t e = hipMemcpyFromSymbol(host, HIP_SYMBOL(g_quant_stamps), static_cast<size_t>(rows) * kStampSlots * sizeof(unsigned long long));
    TPQ_REQUIRE(e == hipSuccess, TPQ_ERR_RUNTIME, "quantize stamps: %s", hipGetErrorString(e));
    return TPQ_OK;
}
#endif

TPQ_EXPORT int tpq_quantize_rowwise(const void* x, int x_dtype, int64_t M, int64_t K, float eps,
                                    float divisor, int qmin, int qmax, int sign_mode,
                                    int8_t* codes, float* scales, void* stream) {
    using namespace tpq;
    TPQ_REQUIRE(M >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "quantize_rowwise: negative shape");
    TPQ_REQUIRE(x_dtype == TPQ_DTYPE_F32 || x_dtype == TPQ_DTYPE_F16 || x_dtype == TPQ_DTYPE_BF16,
                TPQ_ERR_INVALID_TYPE, "rowwise quantize: unsupported input dtype");
    TPQ_REQUIRE(qmin >= -128 && qmax <= 127 && qmin <= qmax && divisor > 0.0f, TPQ_ERR_INVALID_VALUE,
                "quantize_rowwise: code range must fit int8 and divisor must be positive");
    if (M == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(x && codes && scales, TPQ_ERR_INVALID_VALUE, "quantize_rowwise: null pointer");
    TPQ_REQUIRE(M <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "quantize_rowwise: more than 2^31-1 rows");
    // |v| / scale <= divisor (1 + 2^-22) for every element of the row, whatever the rounding of scale and of the quotient
    const float reach = rintf(divisor * (1.0f + 0x1p-20f));
    const int no_clamp = divisor <= 127.0f && reach <= static_cast<float>(qmax) && -reach >= static_cast<float>(qmin);
    const QParams p{eps, divisor, qmin, qmax, sign_mode ? 1 : 0, no_clamp};
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (x_dtype) {
        case TPQ_DTYPE_F32: return launch<TPQ_DTYPE_F32>(x, M, K, p, codes, scales, s);
        case TPQ_DTYPE_F16: return launch<TPQ_DTYPE_F16>(x, M, K, p, codes, scales, s);
        default: return launch<TPQ_DTYPE_BF16>(x, M, K, p, codes, scales, s);
    }
}
