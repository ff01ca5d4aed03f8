// BitNet b1.58 packed linear: int8 activations x 2-bit packed ternary weights.
//
//   acc[m,n] = sum_k x[m,k] * code[n,k],  code = sign-extended 2-bit field
//   out[m,n] = cast((float(acc) * row_scale[m]) * w_scale (+ bias[n]))
//
// The packed matrix [N, ceil(K/4)] is streamed as it is; no int8 copy of the
// weight is ever materialised (the reference unpacks to int8 on every call,
// tensorplay/ao/quantization/bitnet.py:233).
//
// One row, K % 64 == 0, K <= 8192: the flat dot-product kernel of ternary_row_kernel.h.
// Up to 32 rows with K % 256 == 0: the matrix-core decode kernel of ternary_decode_mfma.h.
//
// Dot-product decode kernel (M <= 8, other K % 64 == 0): one wavefront per 4 weight rows, lane l owns the
// 16-byte chunks l, l+64, ... of each row (64 codes per chunk, 1 KB per
// wavefront load).  For field position q of every byte,
//   f = (w >> (6-2q)) & 0x03030303  are four unsigned codes, and
//   sext(f) = f - 4*(f >> 1), so  sum x*code = dot4(x_q, f) - 4*dot4(x_q, f>>1)
// with x_q the activations of that field position gathered into one register
// (a 4x4 byte transpose of the activation chunk, done once per wavefront and
// reused for its rows).  v_dot4_i32_i8 does the multiply-adds.
//
// More rows: the tile kernel of ternary_gemm_kernel.h (K % 256 == 0), else (K % 16 == 0) the int8
// matrix-core GEMM with a loader that expands the 2-bit chunks to int8 on their way into LDS.
//
// Anything else: one thread per output.
#include <cstdlib>

#include "int8_gemm_kernel.h"
#include "ternary_gemm_kernel.h"
#include "ternary_decode_mfma.h"
#include "ternary_row_kernel.h"
#include "ternary_slab_kernel.h"

namespace tpq {
namespace {

constexpr int kRowsPerWave = 4;

template <int MROWS, class Epilogue>
__global__ __launch_bounds__(256) void ternary_decode_kernel(const int8_t* __restrict__ x,
                                                             const uint8_t* __restrict__ packed,
                                                             int m_base, int N, int K, Epilogue ep) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int n0 = wave * kRowsPerWave;
    if (n0 >= N) return;
    const int chunks = K >> 6;  // K % 64 == 0
    const size_t bpr = static_cast<size_t>(K) >> 2;

    int acc_f[kRowsPerWave][MROWS], acc_h[kRowsPerWave][MROWS];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
        for (int m = 0; m < MROWS; ++m) acc_f[r][m] = acc_h[r][m] = 0;

    for (int chunk = lane; chunk < chunks; chunk += kWave) {
        uint4 w[kRowsPerWave];
#pragma unroll
        for (int r = 0; r < kRowsPerWave; ++r) {
            const int n = n0 + r < N ? n0 + r : N - 1;
            w[r] = *reinterpret_cast<const uint4*>(packed + n * bpr + static_cast<size_t>(chunk) * 16);
        }
        // activations of this chunk, regrouped by field position: xq[m][d][q]
        uint32_t xq[MROWS][4][4];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
            const uint4* xp = reinterpret_cast<const uint4*>(x + static_cast<size_t>(m_base + m) * K + static_cast<size_t>(chunk) * 64);
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint4 v = xp[d];
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    xq[m][d][q] = ((v.x >> (8 * q)) & 0xFFu) | (((v.y >> (8 * q)) & 0xFFu) << 8) |
                                  (((v.z >> (8 * q)) & 0xFFu) << 16) | (((v.w >> (8 * q)) & 0xFFu) << 24);
            }
        }
#pragma unroll
        for (int r = 0; r < kRowsPerWave; ++r) {
            const uint32_t wd[4] = {w[r].x, w[r].y, w[r].z, w[r].w};
#pragma unroll
            for (int d = 0; d < 4; ++d)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t f = (wd[d] >> (6 - 2 * q)) & 0x03030303u;
                    const uint32_t h = (wd[d] >> (7 - 2 * q)) & 0x01010101u;
#pragma unroll
                    for (int m = 0; m < MROWS; ++m) {
                        acc_f[r][m] = __builtin_amdgcn_sdot4(static_cast<int>(xq[m][d][q]), static_cast<int>(f), acc_f[r][m], false);
                        acc_h[r][m] = __builtin_amdgcn_sdot4(static_cast<int>(xq[m][d][q]), static_cast<int>(h), acc_h[r][m], false);
                    }
                }
        }
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
            const int total = wave_sum(acc_f[r][m] - 4 * acc_h[r][m]);
            const int n = n0 + r;
            if (lane == 0 && n < N) ep.store(static_cast<int64_t>(m_base + m) * N + n, m_base + m, n, total);
        }
}

template <class Epilogue>
__global__ __launch_bounds__(256) void ternary_generic_kernel(const int8_t* __restrict__ x,
                                                              const uint8_t* __restrict__ packed,
                                                              int64_t M, int64_t N, int64_t K, Epilogue ep) {
    const int64_t bpr = (K + 3) / 4;
    const int64_t total = M * N;
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total; idx += gridDim.x * 256ll) {
        const int64_t m = idx / N, n = idx - m * N;
        int acc = 0;
        for (int64_t k = 0; k < K; ++k) {
            const uint32_t b = static_cast<uint32_t>(packed[n * bpr + (k >> 2)]) << 24;
            const int code = static_cast<int32_t>(b << (2 * (k & 3))) >> 30;
            acc += static_cast<int>(x[m * K + k]) * code;
        }
        ep.store(idx, static_cast<int>(m), static_cast<int>(n), acc);
    }
}

template <class Epilogue>
int launch_ternary(const int8_t* x, const uint8_t* packed, int64_t M, int64_t N, int64_t K,
                   Epilogue ep, hipStream_t s, void* workspace, int64_t workspace_bytes) {
    const bool sizes_ok = M <= 0x7FFFFFFF && N <= 0x7FFFFFFF && K <= 0x7FFFFFFF;
    // the tile kernel below takes over where it is faster and its shape conditions hold
    // Measured at 2560 -> 6912 / 6912 -> 2560 (216 / 80 tiles of 32 channels): the decode kernel takes 7, 7.5, 9.4, 11.4 us
    // for 1..4 rows and twice that for 5..8, the tile kernel 9.3 / 18.3 us for any row count up to 128.
    static const int forced_decode_rows = [] { const char* e = tuning_env("TPQ_TERNARY_DECODE_ROWS"); return e ? std::atoi(e) : -1; }();
    // ... and stays ahead of the 256 x 128-tile kernel at every larger row count tried (512 rows: 30 / 33 us against
    // 54 / 103 us; 2048 rows: 100 / 85 us against 111 / 112 us), so there is no upper limit by default.
    static const int64_t gemm_rows = [] { const char* e = tuning_env("TPQ_TERNARY_GEMM_ROWS"); return e ? std::atoll(e) : int64_t{1} << 40; }();
    const int decode_rows = forced_decode_rows >= 0 ? forced_decode_rows : ((N + kTgN - 1) / kTgN >= 128 ? 3 : 6);
    // Up to 32 rows, in slabs of 16: the weight streamed once per slab through the matrix cores.  Measured against the
    // kernels below over K, N = 1024..28672: one row 4.3..19.8 us (the dot-product kernel 4.7..19.2), 16 rows
    // 5.2..29.6 us (the tile kernel 9.3..75 us for any row count up to 128; two slabs stay below it, three do not).
    static const int mfma_min = [] { const char* e = tuning_env("TPQ_TERNARY_MFMA_MIN"); return e ? std::atoi(e) : 1; }();
    static const int mfma_rows = [] { const char* e = tuning_env("TPQ_TERNARY_MFMA_ROWS"); return e ? std::atoi(e) : 32; }();
    // One row, K up to 8192: the flat dot-product kernel (every wave-level load 1 KB of whole lines)
    if (forced_decode_rows < 0 && M == 1 && aligned(x, 16) && aligned(packed, 16) && !tuning_env("TPQ_TERNARY_NO_ROW")) {
        if (const int rows_wg = ternary_row_rows_per_workgroup(M, N, K)) return launch_ternary_row(x, packed, N, K, rows_wg, ep, s);
    }
    if (forced_decode_rows < 0 && M >= mfma_min && M <= mfma_rows && ternary_decode_mfma_ok(x, packed, M, N, K))
        return launch_ternary_decode_mfma(x, packed, M, N, K, ep, s);
    // 33 rows and more: the slab kernel (every load of a workgroup in flight at once); K beyond 2560 is split and
    // needs the caller's workspace for the exact partial sums
    if (forced_decode_rows < 0 && !tuning_env("TPQ_TERNARY_NO_SLAB") && aligned(x, 16) && aligned(packed, 16)) {
        const int splits = ternary_slab_splits(M, N, K);
        const bool room = splits == 1 || (workspace != nullptr && aligned(workspace, 16) && workspace_bytes >= static_cast<int64_t>(splits) * M * N * 4);
        if (splits >= 1 && room) return launch_ternary_slab(x, packed, M, N, K, splits, static_cast<int32_t*>(workspace), ep, s);
    }
    const bool gemm_ok = sizes_ok && M <= gemm_rows && K % kTgStage == 0 && aligned(x, 16) && aligned(packed, 4);
    if (sizes_ok && M <= 8 && (M <= decode_rows || !gemm_ok) && K % 64 == 0 && aligned(x, 16) && aligned(packed, 16)) {
        const int waves = static_cast<int>((N + kRowsPerWave - 1) / kRowsPerWave);
        const dim3 grid((waves + 3) / 4);
        for (int m0 = 0; m0 < M; m0 += 4) {
            const int rows = static_cast<int>(M - m0 < 4 ? M - m0 : 4);
            switch (rows) {
                case 1: ternary_decode_kernel<1, Epilogue><<<grid, 256, 0, s>>>(x, packed, m0, (int)N, (int)K, ep); break;
                case 2: ternary_decode_kernel<2, Epilogue><<<grid, 256, 0, s>>>(x, packed, m0, (int)N, (int)K, ep); break;
                case 3: ternary_decode_kernel<3, Epilogue><<<grid, 256, 0, s>>>(x, packed, m0, (int)N, (int)K, ep); break;
                default: ternary_decode_kernel<4, Epilogue><<<grid, 256, 0, s>>>(x, packed, m0, (int)N, (int)K, ep); break;
            }
        }
        return check_launch("tpq_ternary_mm (decode)");
    }
    if (gemm_ok) return launch_ternary_gemm_m128(x, packed, M, N, K, ep, s);
    if (sizes_ok && K % 16 == 0 && aligned(x, 16) && aligned(packed, 4))
        return launch_mfma<true>(x, packed, M, N, K, ep, s);
    const int64_t blocks = (M * N + 255) / 256;
    ternary_generic_kernel<Epilogue><<<static_cast<unsigned>(blocks > 65535 ? 65535 : blocks), 256, 0, s>>>(
        x, packed, M, N, K, ep);
    return check_launch("tpq_ternary_mm (generic)");
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int64_t tpq_ternary_mm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const int splits = M > 0 && N > 0 && K > 0 ? ternary_slab_splits(M, N, K) : 0;
    return splits > 1 ? static_cast<int64_t>(splits) * M * N * 4 : 0;
}

TPQ_EXPORT int tpq_ternary_mm(const int8_t* x, const float* row_scale, const uint8_t* packed,
                              float w_scale, const float* bias, int64_t M, int64_t N, int64_t K,
                              void* out, int out_dtype, int32_t* acc_out, void* stream) {
    return tpq_ternary_mm_ws(x, row_scale, packed, w_scale, bias, M, N, K, out, out_dtype, acc_out, nullptr, 0, stream);
}

TPQ_EXPORT int tpq_ternary_mm_ws(const int8_t* x, const float* row_scale, const uint8_t* packed,
                                 float w_scale, const float* bias, int64_t M, int64_t N, int64_t K,
                                 void* out, int out_dtype, int32_t* acc_out, void* workspace, int64_t workspace_bytes,
                                 void* stream) {
    TPQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "bitnet_linear_packed: negative shape");
    TPQ_REQUIRE(out_dtype == TPQ_DTYPE_F32 || out_dtype == TPQ_DTYPE_F16 || out_dtype == TPQ_DTYPE_BF16,
                TPQ_ERR_INVALID_TYPE, "bitnet_linear_packed: unsupported output dtype");
    if (M == 0 || N == 0) return TPQ_OK;
    TPQ_REQUIRE(out || acc_out, TPQ_ERR_INVALID_VALUE, "bitnet_linear_packed: no destination");
    TPQ_REQUIRE((K == 0 || (x && packed)) && (!out || row_scale), TPQ_ERR_INVALID_VALUE,
                "bitnet_linear_packed: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (out_dtype) {
        case TPQ_DTYPE_F32: {
            const EpilogueTernary<TPQ_DTYPE_F32> ep{static_cast<float*>(out), acc_out, row_scale, bias, w_scale};
            return launch_ternary(x, packed, M, N, K, ep, s, workspace, workspace_bytes);
        }
        case TPQ_DTYPE_F16: {
            const EpilogueTernary<TPQ_DTYPE_F16> ep{static_cast<uint16_t*>(out), acc_out, row_scale, bias, w_scale};
            return launch_ternary(x, packed, M, N, K, ep, s, workspace, workspace_bytes);
        }
        default: {
            const EpilogueTernary<TPQ_DTYPE_BF16> ep{static_cast<uint16_t*>(out), acc_out, row_scale, bias, w_scale};
            return launch_ternary(x, packed, M, N, K, ep, s, workspace, workspace_bytes);
        }
    }
}
