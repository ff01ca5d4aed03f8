// rms_norm over the last dimension: out[m][k] = T((x[m][k] * inv[m]) * w[k]), inv = 1 / sqrt(mean(x[m]^2) + eps),
// computed in fp32 and rounded once to the input type, the formulation of the reference's CPU kernel
// (p10/src/backend/cpu/NormalizationKernels.cpp:1355-1453; Python composite tensorplay/nn/functional.py:2350-2372).
//
// HBM-bound: a row is read once and written once.  One workgroup per row holds the row in registers between the
// sum of squares and the scaling (up to 8 x 256 x 8 = 16384 elements; longer rows are read a second time, from
// cache).  The sum of squares is added in a fixed tree order (per thread, across lanes, across wavefronts), which
// differs from the serial fp32 sum of the CPU kernel by rounding only: the result agrees with the reference to an
// ulp of the output type, not bit for bit.  The decode path does not come here: there the norm is folded into the
// matmul that follows it (int4_mfma_flight_kernel.h); this is the op for prefill blocks and for the shapes the
// folded form is not built for.
#include "tpq_common.h"

namespace tpq {
namespace {

constexpr int kNormThreads = 256, kNormMaxChunks = 8;  // chunks of 8 elements per thread held in registers

// The 16-byte chunks (eight elements; fp32: 32 bytes) of a row are dealt to the threads of the workgroup round-robin.
// CHUNKS > 0: the row fits CHUNKS chunks per thread and stays in registers; CHUNKS = 0: any length, second pass re-reads.
template <int DT, int CHUNKS>
__global__ __launch_bounds__(kNormThreads) void rms_norm_rows_kernel(const typename Elem<DT>::storage* __restrict__ x,
                                                                   const typename Elem<DT>::storage* __restrict__ w,
                                                                   typename Elem<DT>::storage* __restrict__ out, int K, float eps) {
    using T = typename Elem<DT>::storage;
    __shared__ float part[kNormThreads / kWave];
    const int tid = threadIdx.x;
    const T* row = x + static_cast<size_t>(blockIdx.x) * K;
    T* dst = out + static_cast<size_t>(blockIdx.x) * K;
    const int n_chunks = K >> 3;
    float v[CHUNKS > 0 ? CHUNKS : 1][8];
    float acc = 0.0f;
    if constexpr (CHUNKS > 0) {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int chunk = tid + c * kNormThreads;
            load_eight<DT>(row + static_cast<size_t>(chunk < n_chunks ? chunk : 0) * 8, v[c]);  // past the end: re-read, not added
        }
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
            if (tid + c * kNormThreads < n_chunks)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(v[c][e], v[c][e], acc);
    } else {
        for (int chunk = tid; chunk < n_chunks; chunk += kNormThreads) {
            load_eight<DT>(row + static_cast<size_t>(chunk) * 8, v[0]);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(v[0][e], v[0][e], acc);
        }
    }
    acc = wave_sum(acc);
    if ((tid & (kWave - 1)) == 0) part[tid >> 6] = acc;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < kNormThreads / kWave; ++i) total += part[i];
    const float inv = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, static_cast<float>(K)), eps)));

    auto finish = [&](int chunk, const float (&xv)[8]) {
        float g[8];
        if (w != nullptr) {
            load_eight<DT>(w + static_cast<size_t>(chunk) * 8, g);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) g[e] = 1.0f;
        }
        float r[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = __fmul_rn(__fmul_rn(xv[e], inv), g[e]);
        if constexpr (DT == TPQ_DTYPE_F32) {
            float4* o = reinterpret_cast<float4*>(dst + static_cast<size_t>(chunk) * 8);
            o[0] = make_float4(r[0], r[1], r[2], r[3]);
            o[1] = make_float4(r[4], r[5], r[6], r[7]);
        } else {
            uint32_t p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                p[i] = static_cast<uint32_t>(Elem<DT>::store(r[2 * i])) | (static_cast<uint32_t>(Elem<DT>::store(r[2 * i + 1])) << 16);
            *reinterpret_cast<uint4*>(dst + static_cast<size_t>(chunk) * 8) = make_uint4(p[0], p[1], p[2], p[3]);
        }
    };
    if constexpr (CHUNKS > 0) {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
            if (tid + c * kNormThreads < n_chunks) finish(tid + c * kNormThreads, v[c]);
    } else {
        for (int chunk = tid; chunk < n_chunks; chunk += kNormThreads) {
            load_eight<DT>(row + static_cast<size_t>(chunk) * 8, v[0]);
            finish(chunk, v[0]);
        }
    }
}

// Rows whose length is not a multiple of eight, or whose pointers are not 16-byte aligned: one element at a time.
template <int DT>
__global__ __launch_bounds__(kNormThreads) void rms_norm_rows_plain_kernel(const typename Elem<DT>::storage* __restrict__ x,
                                                                         const typename Elem<DT>::storage* __restrict__ w,
                                                                         typename Elem<DT>::storage* __restrict__ out, int K, float eps) {
    __shared__ float part[kNormThreads / kWave];
    const int tid = threadIdx.x;
    const auto* row = x + static_cast<size_t>(blockIdx.x) * K;
    auto* dst = out + static_cast<size_t>(blockIdx.x) * K;
    float acc = 0.0f;
    for (int k = tid; k < K; k += kNormThreads) {
        const float v = Elem<DT>::load(row[k]);
        acc = __builtin_fmaf(v, v, acc);
    }
    acc = wave_sum(acc);
    if ((tid & (kWave - 1)) == 0) part[tid >> 6] = acc;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < kNormThreads / kWave; ++i) total += part[i];
    const float inv = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, static_cast<float>(K)), eps)));
    for (int k = tid; k < K; k += kNormThreads) {
        const float g = w != nullptr ? Elem<DT>::load(w[k]) : 1.0f;
        dst[k] = Elem<DT>::store(__fmul_rn(__fmul_rn(Elem<DT>::load(row[k]), inv), g));
    }
}

template <int DT>
int launch(const void* x, const void* w, void* out, int64_t M, int64_t K, float eps, hipStream_t s) {
    using T = typename Elem<DT>::storage;
    const auto* xp = static_cast<const T*>(x);
    const auto* wp = static_cast<const T*>(w);
    auto* op = static_cast<T*>(out);
    const dim3 grid(static_cast<unsigned>(M)), block(kNormThreads);
    const int k = static_cast<int>(K);
    const bool vector_ok = K % 8 == 0 && aligned(x, 16) && aligned(out, 16) && (w == nullptr || aligned(w, 16));
    if (!vector_ok) {
        rms_norm_rows_plain_kernel<DT><<<grid, block, 0, s>>>(xp, wp, op, k, eps);
        return check_launch("tpq_rms_norm");
    }
    const int64_t per_thread = (K / 8 + kNormThreads - 1) / kNormThreads;
    if (per_thread <= 1) rms_norm_rows_kernel<DT, 1><<<grid, block, 0, s>>>(xp, wp, op, k, eps);
    else if (per_thread <= 2) rms_norm_rows_kernel<DT, 2><<<grid, block, 0, s>>>(xp, wp, op, k, eps);
    else if (per_thread <= 4) rms_norm_rows_kernel<DT, 4><<<grid, block, 0, s>>>(xp, wp, op, k, eps);
    else if (per_thread <= kNormMaxChunks) rms_norm_rows_kernel<DT, kNormMaxChunks><<<grid, block, 0, s>>>(xp, wp, op, k, eps);
    else rms_norm_rows_kernel<DT, 0><<<grid, block, 0, s>>>(xp, wp, op, k, eps);
    return check_launch("tpq_rms_norm");
}

}  // namespace
}  // namespace tpq

TPQ_EXPORT int tpq_rms_norm(const void* x, int dtype, int64_t M, int64_t K, const void* weight, float eps, void* out, void* stream) {
    using namespace tpq;
    TPQ_REQUIRE(M >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "rms_norm: negative shape");
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F32 || dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16, TPQ_ERR_INVALID_TYPE,
                "rms_norm: unsupported dtype");
    if (M == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(x && out, TPQ_ERR_INVALID_VALUE, "rms_norm: null pointer");
    TPQ_REQUIRE(M <= 0x7FFFFFFF && K <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "rms_norm: more than 2^31-1 rows or columns");
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case TPQ_DTYPE_F32: return launch<TPQ_DTYPE_F32>(x, weight, out, M, K, eps, s);
        case TPQ_DTYPE_F16: return launch<TPQ_DTYPE_F16>(x, weight, out, M, K, eps, s);
        default: return launch<TPQ_DTYPE_BF16>(x, weight, out, M, K, eps, s);
    }
}
