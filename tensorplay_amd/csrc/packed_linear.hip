// The linear, float-output form of the reference's prepacked quantized operator
// (_quantized_packed_run: p10/src/backend/cpu/QuantPacked.cpp:420-516, 537-572; packed_real_value:
// p10/include/QuantPacked.h:133-139) for per-tensor quantized activations and per-channel quantized weights:
//   acc[m][n] = sum_k x[m][k] w[n][k] - xz off[n] - wz[n] sum_k x[m][k] + K xz wz[n]        (integers, exact)
//   out[m][n] = fmaf(float(acc), float(xs) * ws[n], bias[n] or 0)   (relu: max(out, 0))
// with off[n] = sum_k w[n][k], the offsets the prepack stores (_quantized_weight_prepack, QuantPacked.cpp:519-533).
//
// Two launches: the int32 products through tpq_int_mm (MFMA-bound at many rows, HBM-bound at few; unsigned activations
// are first turned into signed ones, x - 128, so that they take the matrix-core kernels too: the 128 off[n] that this
// leaves out is added back with the other integer terms), then one pass that adds the rows of x, applies the integer
// corrections in 64 bits and the float epilogue.  The hot path of the int8 linears calls the operator with unit scales
// and zero zero-points, where it reduces to float(tpq_int_mm).
#include "tpq_common.h"

namespace tpq {
namespace {

__global__ __launch_bounds__(256) void flip_sign_kernel(const uint32_t* __restrict__ in, uint32_t* __restrict__ out, int64_t words) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < words; i += stride) out[i] = in[i] ^ 0x80808080u;
}
__global__ __launch_bounds__(256) void flip_sign_bytes_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int64_t first, int64_t bytes) {
    const int64_t i = first + static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < bytes) out[i] = in[i] ^ 0x80u;
}

constexpr int kFinishColumns = 2048;  // columns per workgroup: the row of x is added up once per workgroup

// grid (M, ceil(N / kFinishColumns)); flipped: the products were formed with x - 128
__global__ __launch_bounds__(256) void packed_finish_kernel(const int32_t* __restrict__ acc, const void* __restrict__ x, int x_unsigned,
                                                           float xs, long long xz, const long long* __restrict__ offsets,
                                                           const float* __restrict__ ws, const long long* __restrict__ wz,
                                                           const float* __restrict__ bias, int relu, int flipped,
                                                           float* __restrict__ out, int64_t N, int64_t K) {
    __shared__ long long part[256 / kWave];
    const int64_t m = blockIdx.x;
    const int tid = threadIdx.x;
    long long sum = 0;
    if (x_unsigned) {
        const uint8_t* row = static_cast<const uint8_t*>(x) + m * K;
        for (int64_t k = tid; k < K; k += 256) sum += row[k];
    } else {
        const int8_t* row = static_cast<const int8_t*>(x) + m * K;
        for (int64_t k = tid; k < K; k += 256) sum += row[k];
    }
#pragma unroll
    for (int off = kWave / 2; off >= 1; off >>= 1) {
        const int lo = __shfl_xor(static_cast<int>(sum & 0xFFFFFFFFll), off, kWave);
        const int hi = __shfl_xor(static_cast<int>(sum >> 32), off, kWave);
        sum += (static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo);
    }
    if ((tid & (kWave - 1)) == 0) part[tid >> 6] = sum;
    __syncthreads();
    long long row_sum = 0;
#pragma unroll
    for (int w = 0; w < 256 / kWave; ++w) row_sum += part[w];

    const int64_t n0 = static_cast<int64_t>(blockIdx.y) * kFinishColumns;
    const int64_t n1 = n0 + kFinishColumns < N ? n0 + kFinishColumns : N;
    for (int64_t n = n0 + tid; n < n1; n += 256) {
        long long raw = acc[m * N + n];
        if (flipped) raw += 128ll * offsets[n];
        const long long z = wz[n];
        const long long a = raw - xz * offsets[n] - z * row_sum + static_cast<long long>(K) * xz * z;
        float v = __builtin_fmaf(static_cast<float>(a), __fmul_rn(xs, ws[n]), bias ? bias[n] : 0.0f);
        if (relu) v = v > 0.0f ? v : 0.0f;  // the reference: max(value, 0.) on the double of this float
        out[m * N + n] = v;
    }
}

size_t round_up16(size_t v) { return (v + 15) & ~static_cast<size_t>(15); }

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT size_t tpq_packed_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int x_unsigned) {
    if (M <= 0 || N <= 0) return 0;
    size_t bytes = round_up16(static_cast<size_t>(M) * static_cast<size_t>(N) * sizeof(int32_t));
    if (x_unsigned && K > 0) bytes += round_up16(static_cast<size_t>(M) * static_cast<size_t>(K));
    return bytes;
}

TPQ_EXPORT int tpq_packed_linear_float(const void* x, int x_unsigned, double x_scale, int64_t x_zero_point, const int8_t* packed,
                                       int64_t packed_row_stride, const int64_t* offsets, const float* w_scales,
                                       const int64_t* w_zero_points, const float* bias, int relu, float* out, int64_t M, int64_t N,
                                       int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
    TPQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "packed linear: negative shape");
    if (M == 0 || N == 0) return TPQ_OK;
    TPQ_REQUIRE(out && offsets && w_scales && w_zero_points && (K == 0 || (x && packed)), TPQ_ERR_INVALID_VALUE, "packed linear: null pointer");
    TPQ_REQUIRE(packed_row_stride >= K, TPQ_ERR_INVALID_VALUE, "packed linear: the rows of the packed weight are shorter than K");
    // |x| <= 255, |w| <= 128: the int32 products of tpq_int_mm hold up to this K
    TPQ_REQUIRE(K <= 65536, TPQ_ERR_UNSUPPORTED, "packed linear: K above 65536 is not built");
    TPQ_REQUIRE(M <= 0x7FFFFFFF && N <= 65535ll * kFinishColumns, TPQ_ERR_UNSUPPORTED, "packed linear: more rows or channels than the finishing launch's grid holds");
    TPQ_REQUIRE(workspace && aligned(workspace, 16) && workspace_bytes >= tpq_packed_linear_workspace_bytes(M, N, K, x_unsigned),
                TPQ_ERR_INVALID_VALUE, "packed linear: workspace of tpq_packed_linear_workspace_bytes(M, N, K, x_unsigned) bytes needed");
    hipStream_t s = static_cast<hipStream_t>(stream);
    int32_t* acc = static_cast<int32_t*>(workspace);
    const void* lhs = x;
    int lhs_unsigned = x_unsigned;
    int flipped = 0;
    if (x_unsigned && K > 0) {  // x - 128 as int8, so that the product runs on the signed kernels
        uint8_t* xf = static_cast<uint8_t*>(workspace) + round_up16(static_cast<size_t>(M) * N * sizeof(int32_t));
        const int64_t bytes = M * K, words = aligned(x, 4) ? bytes / 4 : 0;
        if (words) {
            const int64_t blocks = (words + 255) / 256;
            flip_sign_kernel<<<static_cast<unsigned>(blocks > 4096 ? 4096 : blocks), 256, 0, s>>>(static_cast<const uint32_t*>(x), reinterpret_cast<uint32_t*>(xf), words);
        }
        if (bytes > words * 4) {
            const int64_t rest = bytes - words * 4;
            flip_sign_bytes_kernel<<<static_cast<unsigned>((rest + 255) / 256), 256, 0, s>>>(static_cast<const uint8_t*>(x), xf, words * 4, bytes);
        }
        if (int rc = check_launch("packed linear (signed copy of the activations)")) return rc;
        lhs = xf;
        lhs_unsigned = 0;
        flipped = 1;
    }
    if (int rc = tpq_int_mm(lhs, lhs_unsigned, packed, 1, packed_row_stride, acc, M, K, N, stream)) return rc;
    const dim3 grid(static_cast<unsigned>(M), static_cast<unsigned>((N + kFinishColumns - 1) / kFinishColumns));
    packed_finish_kernel<<<grid, 256, 0, s>>>(acc, x, x_unsigned, static_cast<float>(x_scale), static_cast<long long>(x_zero_point),
                                              reinterpret_cast<const long long*>(offsets), w_scales,
                                              reinterpret_cast<const long long*>(w_zero_points), bias, relu, flipped, out, N, K);
    return check_launch("packed linear (corrections and epilogue)");
}
