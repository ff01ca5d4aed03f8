// out[M][N] = x[M][K] w[N][K]^T for float16 / bfloat16 / float32 operands, float32 accumulation, one rounding to the
// operand type: the plain GEMM behind the reference's "dequantise the weight, then multiply" route for many activation rows
// (p10/src/backend/cuda/QuantGemmKernels.cu:1339 gemm_impl(xf, wf.t(), out, 1.0, 0.0, nullptr); the same step in
// _weight_int8pack_mm and the low-bit linear).  The callers dequantise the packed weight into a dense [N][K] matrix
// first (tpq_int4_dequantize and its siblings) and come here with it.
//
// MFMA-bound: 2 M N K flops.  The kernel is the staggered tile kernel of the int8 GEMM (gemm_stagger.h) with
// v_mfma_f32_16x16x32_f16 / _bf16 (or four v_mfma_f32_16x16x4_f32) in place of the int8 instruction: a stage is 128
// bytes = 64 (32) elements of k per row.
#include "gemm_stagger.h"

namespace tpq {
namespace {

constexpr double kShortTile = 0.8;

template <int DT, class Arith>
int dense_mm_typed(const void* x, const void* w, void* out, int64_t M, int64_t N, int64_t K, hipStream_t s) {
    const TileFloat<DT> tile{static_cast<typename Elem<DT>::storage*>(out), nullptr, nullptr, nullptr};
    // Tile height: whole rounds of tiles over the 256 compute units, a 128-row tile costing kShortTile of a 256-row one
    // (its stages are bound by the loads, not by the MFMAs).
    const int64_t tiles_n = (N + 127) / 128, units = 256;
    const int64_t rounds_tall = (((M + 255) / 256) * tiles_n + units - 1) / units, rounds_short = (((M + 127) / 128) * tiles_n + units - 1) / units;
    const char* env = tuning_env("TPQ_DENSE_TILE");
    const bool use_short = env ? env[0] == 's' : static_cast<double>(rounds_short) * kShortTile < static_cast<double>(rounds_tall);
    constexpr int64_t kElem = sizeof(typename Elem<DT>::storage);
    if (use_short) return launch_stagger_bytes<Arith, 2>(x, w, M, N, K * kElem, tile, s, 1, "dense gemm (staggered, 128 rows)");
    return launch_stagger_bytes<Arith, 4>(x, w, M, N, K * kElem, tile, s, 1, "dense gemm (staggered)");
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int tpq_dense_mm(const void* x, int dtype, int64_t M, int64_t K, const void* w, int64_t N, void* out, void* stream) {
    TPQ_REQUIRE(dtype == TPQ_DTYPE_F16 || dtype == TPQ_DTYPE_BF16 || dtype == TPQ_DTYPE_F32, TPQ_ERR_UNSUPPORTED,
                "tpq_dense_mm: float16 / bfloat16 / float32 operands only");
    TPQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "tpq_dense_mm: negative dimension");
    if (M == 0 || N == 0) return TPQ_OK;
    const int64_t per_stage = dtype == TPQ_DTYPE_F32 ? 32 : 64;  // elements of k in the 128 bytes of a stage
    TPQ_REQUIRE(K > 0 && K % per_stage == 0 && K * (128 / per_stage) < (1 << 23), TPQ_ERR_UNSUPPORTED,
                "tpq_dense_mm: K must be a positive multiple of 64 (float32: 32), a row below 8 MB");
    TPQ_REQUIRE(M <= 0x7FFFFFFF && N <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "tpq_dense_mm: dimension too large");
    TPQ_REQUIRE(x && w && out, TPQ_ERR_INVALID_VALUE, "tpq_dense_mm: null pointer");
    TPQ_REQUIRE(aligned(x, 16) && aligned(w, 16) && aligned(out, dtype == TPQ_DTYPE_F32 ? 4 : 2), TPQ_ERR_INVALID_VALUE,
                "tpq_dense_mm: x and w must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == TPQ_DTYPE_F32) return dense_mm_typed<TPQ_DTYPE_F32, ArithF32>(x, w, out, M, N, K, s);
    if (dtype == TPQ_DTYPE_F16) return dense_mm_typed<TPQ_DTYPE_F16, ArithF16>(x, w, out, M, N, K, s);
    return dense_mm_typed<TPQ_DTYPE_BF16, ArithBF16>(x, w, out, M, N, K, s);
}
