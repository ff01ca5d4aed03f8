// Registers the gfx950 kernels of libtpq_gfx950.so as TensorPlay's CUDA-key kernels of the quantized-linear ops.
//
// Where it goes: this one translation unit is added to a TensorPlay source tree (or built out of tree with
// tensorplay.utils.cpp_extension.load, which links libp10) together with -ltpq_gfx950.  HIP builds of TensorPlay
// dispatch GPU tensors on the CUDA key, and a later registration overwrites the slot
// (p10/src/Dispatcher.cpp:35-48), so loading this library after libp10 replaces the kernels that
// p10/src/backend/cuda/{QuantGemmKernels,IntMM,LowBitGemmKernels,AffineQuantKernels}.cu registered.
//
// Every function below has exactly the C++ signature of the kernel it replaces, because callers cast the slot
// back to the signature generated from config/native_functions.yaml (p10/include/Dispatcher.h:243-249) and the
// typed registerKernel records typeid of the function pointer (Dispatcher.h:129-135).  Argument checks, output
// allocation, zero-size returns and exception types follow the replaced kernels; the arithmetic is the library's.
//
// Not compiled in this repository: p10/include/Tensor.h:365 includes a header that the reference's code
// generator writes at build time, so the reference's headers do not pass even a syntax-only compile from a plain
// checkout.  tests/test_integration_registrar.py checks what can be checked as text: op names against the yaml,
// signatures against the replaced kernels, and every tpq_* call against include/tpq.h.
#include "Tensor.h"
#include "Dispatcher.h"
#include "Exception.h"
#include "CUDARuntime.h"
#include "Utils.h"
#include "CudaGemm.h"

#include <cstdint>
#include <optional>
#include <string>
#include <tuple>
#include <vector>

#include "tpq.h"

namespace tensorplay {
namespace tpq_gfx950 {
namespace {

// The stream the reference's own kernels launch on; its id is the raw stream handle (CUDARuntime.h:47).
void* current_stream() { return reinterpret_cast<void*>(cuda::getCurrentCUDAStream().id()); }

// Non-zero status of a tpq_* call -> the exception type the reference raises for the same condition.
void check(int status) {
    if (status == TPQ_OK) return;
    const std::string what = tpq_last_error();
    switch (status) {
        case TPQ_ERR_INVALID_VALUE: TP_THROW(ValueError, what);
        case TPQ_ERR_INVALID_TYPE: TP_THROW(TypeError, what);
        case TPQ_ERR_UNSUPPORTED: TP_THROW(NotImplementedError, what);
        default: TP_THROW(RuntimeError, what);
    }
}

int float_tag(DType dtype, const char* op) {
    switch (dtype) {
        case DType::Float32: return TPQ_DTYPE_F32;
        case DType::Float16: return TPQ_DTYPE_F16;
        case DType::BFloat16: return TPQ_DTYPE_BF16;
        default: TP_THROW(TypeError, std::string(op) + "(): unsupported floating dtype");
    }
}

// ---- row-wise quantizers: _quantize_{int8,int4,int2,binary}_rowwise(Tensor self, float eps) -> (Tensor, Tensor) ----
// replaces QuantGemmKernels.cu:1573-1609 and LowBitGemmKernels.cu:115-156
std::tuple<Tensor, Tensor> quantize_rowwise(const Tensor& self, double eps, float divisor, int qmin, int qmax,
                                            int sign_mode, const char* op) {
    if (self.dim() != 2) TP_THROW(ValueError, std::string(op) + "(): expected a 2-D tensor");
    const int64_t M = self.size(0), K = self.size(1);
    const Tensor x = self.contiguous();
    Tensor codes = Tensor::empty({M, K}, DType::Int8, self.device());
    Tensor scales = Tensor::empty({M}, DType::Float32, self.device());
    if (M == 0 || K == 0) return {codes, scales};
    check(tpq_quantize_rowwise(x.data_ptr(), float_tag(x.dtype(), op), M, K, static_cast<float>(eps), divisor, qmin, qmax,
                               sign_mode, static_cast<int8_t*>(codes.data_ptr()), static_cast<float*>(scales.data_ptr()),
                               current_stream()));
    return {codes, scales};
}
std::tuple<Tensor, Tensor> quantize_int8_rowwise(const Tensor& self, double eps) {
    return quantize_rowwise(self, eps, 127.0f, -127, 127, 0, "_quantize_int8_rowwise");
}
std::tuple<Tensor, Tensor> quantize_int4_rowwise(const Tensor& self, double eps) {
    return quantize_rowwise(self, eps, 7.0f, -8, 7, 0, "_quantize_int4_rowwise");
}
std::tuple<Tensor, Tensor> quantize_int2_rowwise(const Tensor& self, double eps) {
    return quantize_rowwise(self, eps, 2.0f, -2, 1, 0, "_quantize_int2_rowwise");
}
std::tuple<Tensor, Tensor> quantize_binary_rowwise(const Tensor& self, double eps) {
    return quantize_rowwise(self, eps, 1.0f, -1, 1, 1, "_quantize_binary_rowwise");
}

// ---- _int8_mm_rescale(Tensor out, Tensor row_scale, Tensor col_scale) -> Tensor; replaces QuantGemmKernels.cu:1625-1650
Tensor int8_mm_rescale(const Tensor& out, const Tensor& row_scale, const Tensor& col_scale) {
    if (out.dim() != 2 || out.dtype() != DType::Int32) TP_THROW(ValueError, "_int8_mm_rescale(): expected a 2-D int32 output");
    const int64_t M = out.size(0), N = out.size(1);
    Tensor result = Tensor::empty({M, N}, DType::Float32, out.device());
    if (M == 0 || N == 0) return result;
    const Tensor acc = out.contiguous();
    const Tensor rs = row_scale.to(DType::Float32).contiguous(), cs = col_scale.to(DType::Float32).contiguous();
    if (rs.numel() != M || cs.numel() != N) TP_THROW(ValueError, "_int8_mm_rescale(): scale lengths do not match the output");
    check(tpq_int8_mm_rescale(static_cast<const int32_t*>(acc.data_ptr()), static_cast<const float*>(rs.data_ptr()),
                              static_cast<const float*>(cs.data_ptr()), static_cast<float*>(result.data_ptr()), M, N,
                              current_stream()));
    return result;
}

// ---- _int_mm(Tensor self, Tensor mat2) -> Tensor and _int_mm.out; replaces IntMM.cu:383-477 ----
void check_int_mm_operands(const Tensor& self, const Tensor& mat2) {
    TP_CHECK(self.dim() == 2 && mat2.dim() == 2, "_int_mm: expected two matrices");
    TP_CHECK(self.size(1) == mat2.size(0), "_int_mm: inner dimensions differ");
    TP_CHECK(self.dtype() == DType::Int8 || self.dtype() == DType::UInt8, "_int_mm: expected the left operand to be int8 or uint8");
    TP_CHECK(mat2.dtype() == DType::Int8, "_int_mm: expected the right operand to be int8");
}
// out: contiguous int32 [M, N].  mat2 is read through its strides: the transposed view of a contiguous [N, K]
// weight (strides 1, K), which the callers pass (tensorplay/ao/quantization/int8_mixed_precision.py:69), needs no copy.
void int_mm_into(const Tensor& self, const Tensor& mat2, Tensor& out) {
    const int64_t M = self.size(0), K = self.size(1), N = mat2.size(1);
    if (out.numel() == 0) return;
    const Tensor lhs = self.contiguous();
    check(tpq_int_mm(lhs.data_ptr(), self.dtype() == DType::UInt8 ? 1 : 0, static_cast<const int8_t*>(mat2.data_ptr()),
                     mat2.stride(0), mat2.stride(1), static_cast<int32_t*>(out.data_ptr()), M, K, N, current_stream()));
}
Tensor int_mm(const Tensor& self, const Tensor& mat2) {
    check_int_mm_operands(self, mat2);
    Tensor out = Tensor::empty({self.size(0), mat2.size(1)}, DType::Int32, self.device());
    int_mm_into(self, mat2, out);
    return out;
}
Tensor& int_mm_out(const Tensor& self, const Tensor& mat2, Tensor& out) {
    check_int_mm_operands(self, mat2);
    TP_CHECK(out.dtype() == DType::Int32, "_int_mm: expected an int32 destination");
    const std::vector<int64_t> target{self.size(0), mat2.size(1)};
    if (static_cast<std::vector<int64_t>>(out.shape()) != target) out.resize_(target);
    if (out.numel() == 0) return out;
    if (out.is_contiguous()) {
        int_mm_into(self, mat2, out);
        return out;
    }
    Tensor value = Tensor::empty(target, DType::Int32, self.device());
    int_mm_into(self, mat2, value);
    out.copy_(value);
    return out;
}

// ---- _convert_weight_to_int4pack(Tensor self, int innerKTiles) -> Tensor; replaces QuantGemmKernels.cu:1349-1408 ----
Tensor convert_weight_to_int4pack(const Tensor& self, int64_t inner_tiles) {
    if (self.dim() != 2) TP_THROW(ValueError, "_convert_weight_to_int4pack(): expected 2-D codes [N,K]");
    if (inner_tiles != 2 && inner_tiles != 4 && inner_tiles != 8)
        TP_THROW(ValueError, "_convert_weight_to_int4pack(): innerKTiles must be 2, 4 or 8");
    const int64_t N = self.size(0), K = self.size(1);
    if (K % 2 != 0) TP_THROW(ValueError, "_convert_weight_to_int4pack(): K must be even");
    const int64_t n_tiles = divUp(N, 8), k_super = divUp(K, inner_tiles * 16);
    Tensor packed = Tensor::empty({n_tiles, k_super, 32, inner_tiles / 2}, DType::Int32, self.device());
    if (N == 0 || K == 0) return packed;
    const Tensor codes = self.to(DType::Int32).contiguous();
    check(tpq_int4_pack(static_cast<const int32_t*>(codes.data_ptr()), N, K, static_cast<int>(inner_tiles),
                        static_cast<int32_t*>(packed.data_ptr()), current_stream()));
    return packed;
}

// ---- _weight_int4pack_mm(Tensor self, Tensor mat2, int qGroupSize, Tensor qScaleAndZeros) -> Tensor ----
// replaces QuantGemmKernels.cu:1210-1341 (same checks, :1216-1257)
Tensor weight_int4pack_mm(const Tensor& self, const Tensor& mat2, int64_t q_group_size, const Tensor& q_scale_and_zeros) {
    if (mat2.dtype() != DType::Int32 || mat2.dim() != 4)
        TP_THROW(TypeError, "_weight_int4pack_mm(): packed weight must be 4-D int32 in the tensor-core B layout");
    if (self.dim() != 2) TP_THROW(ValueError, "_weight_int4pack_mm(): expected 2-D activations [m,k]");
    if (!isFloatingType(self.dtype())) TP_THROW(TypeError, "_weight_int4pack_mm(): activations must be floating point");
    if (q_group_size != 32 && q_group_size != 64 && q_group_size != 128)
        TP_THROW(ValueError, "_weight_int4pack_mm(): qGroupSize must be 32, 64 or 128");
    const int64_t m = self.size(0), k = self.size(1);
    const int64_t k_super = mat2.size(1), inner = mat2.size(3) * 2, n = mat2.size(0) * 8;
    if (mat2.size(2) != 32 || (inner != 2 && inner != 4 && inner != 8))
        TP_THROW(ValueError, "_weight_int4pack_mm(): packed weight layout is invalid");
    if (k_super != divUp(k, inner * 16)) TP_THROW(ValueError, "_weight_int4pack_mm(): K dimension does not match packed B");
    const int64_t groups = divUp(k, q_group_size);
    if (q_scale_and_zeros.dim() != 3 || q_scale_and_zeros.size(0) != groups || q_scale_and_zeros.size(1) != n ||
        q_scale_and_zeros.size(2) != 2)
        TP_THROW(ValueError, "_weight_int4pack_mm(): qScaleAndZeros must be [K/group, N, 2]");
    Tensor out = Tensor::empty({m, n}, self.dtype(), self.device());
    if (m == 0 || n == 0 || k == 0) return out;
    const Tensor x = self.contiguous(), w = mat2.contiguous();
    const Tensor sz = q_scale_and_zeros.to(self.dtype()).contiguous();  // the reference casts them too (:1303)
    const int tag = float_tag(x.dtype(), "_weight_int4pack_mm");
    // Many activation rows: the reference's own formulation (:1296-1341), dense weight in the activation dtype and
    // its library GEMM, with the library's dequantize pass.  Fewer rows: the kernels that stream the packed weight.
    const int64_t dense_rows = x.dtype() == DType::Float32 ? 4 : 256;
    if (inner == 2 && m > dense_rows) {
        Tensor dense = Tensor::empty({n, k}, self.dtype(), self.device());
        check(tpq_int4_dequantize(static_cast<const int32_t*>(w.data_ptr()), 2, n, k, q_group_size, sz.data_ptr(), tag,
                                  dense.data_ptr(), current_stream()));
        cuda::gemm_impl(x, dense.t(), out, 1.0, 0.0, nullptr);
        return out;
    }
    check(tpq_int4_mm(x.data_ptr(), tag, m, k, static_cast<const int32_t*>(w.data_ptr()), static_cast<int>(inner), n,
                      q_group_size, sz.data_ptr(), out.data_ptr(), current_stream()));
    return out;
}

// ---- _weight_int8pack_mm(Tensor self, Tensor mat2, Tensor scales) -> Tensor; replaces QuantGemmKernels.cu:345-405 ----
Tensor weight_int8pack_mm(const Tensor& self, const Tensor& mat2, const Tensor& scales) {
    if (mat2.dtype() != DType::QInt8) TP_THROW(TypeError, "_weight_int8pack_mm(): weight must be QInt8");
    if (self.dim() != 2 || mat2.dim() != 2 || scales.dim() != 1)
        TP_THROW(ValueError, "_weight_int8pack_mm(): expected 2-D activations [B,K], 2-D weight [N,K] and 1-D scales [N]");
    if (!isFloatingType(self.dtype())) TP_THROW(TypeError, "_weight_int8pack_mm(): activations must be floating point");
    const int64_t B = self.size(0), K = self.size(1), N = mat2.size(0);
    if (mat2.size(1) != K) TP_THROW(ValueError, "_weight_int8pack_mm(): K dimension mismatch");
    if (scales.size(0) != N) TP_THROW(ValueError, "_weight_int8pack_mm(): scales length mismatch");
    Tensor out = Tensor::empty({B, N}, self.dtype(), self.device());
    if (N == 0 || B == 0 || K == 0) return out;
    const Tensor x = self.contiguous(), w = mat2.contiguous();
    const Tensor sc = scales.to(DType::Float32).contiguous();
    check(tpq_weight_int8pack_mm(x.data_ptr(), float_tag(x.dtype(), "_weight_int8pack_mm"), B, K,
                                 static_cast<const int8_t*>(w.data_ptr()), static_cast<const float*>(sc.data_ptr()), N,
                                 out.data_ptr(), current_stream()));
    return out;
}

// ---- quantize_affine / dequantize_affine; replace AffineQuantKernels.cu:942-1302 ----
int storage_tag(DType dtype, const char* op) {
    switch (dtype) {
        case DType::QInt8: return TPQ_STORAGE_I8;
        case DType::QUInt8: return TPQ_STORAGE_U8;
        case DType::QInt32: return TPQ_STORAGE_I32;
        case DType::QUInt4x2: return TPQ_STORAGE_U4X2;
        case DType::QUInt2x4: return TPQ_STORAGE_U2X4;
        case DType::QUInt1x8: return TPQ_STORAGE_U1X8;
        default: TP_THROW(TypeError, std::string(op) + "(): unsupported quantized dtype");
    }
}
struct AffineParams {
    Tensor scales, zeros;
    const float* zero_ptr = nullptr;
    int64_t n_scales = 0, n_zeros = 0;
};
AffineParams affine_params(const Tensor& like, const Tensor& scales, const std::optional<Tensor>& zero_points, const char* op) {
    AffineParams p;
    if (scales.device() != like.device() ||
        (zero_points.has_value() && zero_points->numel() > 0 && zero_points->device() != like.device()))
        TP_THROW(RuntimeError, std::string(op) + "(): scales and zero_points must be on the input device");
    p.scales = scales.to(DType::Float32).contiguous();
    p.n_scales = p.scales.numel();
    if (zero_points.has_value() && zero_points->numel() > 0) {
        p.zeros = zero_points->to(DType::Float32).contiguous();
        p.n_zeros = p.zeros.numel();
        p.zero_ptr = static_cast<const float*>(p.zeros.data_ptr());
    }
    return p;
}
Tensor quantize_affine(const Tensor& self, const std::vector<int64_t>& block_size, const Tensor& scales,
                       const std::optional<Tensor>& zero_points, DType dtype, int64_t quant_min, int64_t quant_max) {
    if (!isQuantizedType(dtype)) TP_THROW(TypeError, "quantize_affine(): expected a quantized dtype");
    if (static_cast<int64_t>(block_size.size()) != self.dim())
        TP_THROW(ValueError, "quantize_affine(): block_size rank must match the input rank");
    // float64 input, which the replaced kernel accepts, is narrowed first: the library reads f32 / f16 / bf16
    const Tensor input = (self.dtype() == DType::Float64 ? self.to(DType::Float32) : self).contiguous();
    const std::vector<int64_t> sizes = static_cast<std::vector<int64_t>>(input.shape());
    Tensor out = Tensor::empty(sizes, dtype, self.device());
    if (input.numel() == 0) return out;
    const AffineParams p = affine_params(self, scales, zero_points, "quantize_affine");
    check(tpq_quantize_affine(input.data_ptr(), float_tag(input.dtype(), "quantize_affine"), static_cast<int>(sizes.size()),
                              sizes.data(), block_size.data(), static_cast<const float*>(p.scales.data_ptr()), p.n_scales,
                              p.zero_ptr, p.n_zeros, storage_tag(dtype, "quantize_affine"), quant_min, quant_max,
                              out.data_ptr(), current_stream()));
    return out;
}
Tensor dequantize_affine(const Tensor& self, const std::vector<int64_t>& block_size, const Tensor& scales,
                         const std::optional<Tensor>& zero_points) {
    if (!isQuantizedType(self.dtype())) TP_THROW(TypeError, "dequantize_affine(): expected a quantized tensor");
    if (static_cast<int64_t>(block_size.size()) != self.dim())
        TP_THROW(ValueError, "dequantize_affine(): block_size rank must match the input rank");
    const Tensor codes = self.contiguous();
    const std::vector<int64_t> sizes = static_cast<std::vector<int64_t>>(codes.shape());
    Tensor out = Tensor::empty(sizes, DType::Float32, self.device());
    if (codes.numel() == 0) return out;
    const AffineParams p = affine_params(self, scales, zero_points, "dequantize_affine");
    check(tpq_dequantize_affine(codes.data_ptr(), storage_tag(self.dtype(), "dequantize_affine"), static_cast<int>(sizes.size()),
                                sizes.data(), block_size.data(), static_cast<const float*>(p.scales.data_ptr()), p.n_scales,
                                p.zero_ptr, p.n_zeros, static_cast<float*>(out.data_ptr()), current_stream()));
    return out;
}

// Same form as the reference's own registrations (p10/src/backend/cuda/QuantGemmKernels.cu:1652-1659,
// IntMM.cu:479-482, LowBitGemmKernels.cu:158-161, AffineQuantKernels.cu:1745-1753): bare op names, CUDA key.
TENSORPLAY_LIBRARY_IMPL(CUDA, TpqGfx950Kernels) {
    m.impl("_quantize_int8_rowwise", quantize_int8_rowwise);
    m.impl("_quantize_int4_rowwise", quantize_int4_rowwise);
    m.impl("_quantize_int2_rowwise", quantize_int2_rowwise);
    m.impl("_quantize_binary_rowwise", quantize_binary_rowwise);
    m.impl("_int8_mm_rescale", int8_mm_rescale);
    m.impl("_int_mm", int_mm);
    m.impl("_int_mm.out", int_mm_out);
    m.impl("_convert_weight_to_int4pack", convert_weight_to_int4pack);
    m.impl("_weight_int4pack_mm", weight_int4pack_mm);
    m.impl("_weight_int8pack_mm", weight_int8pack_mm);
    m.impl("quantize_affine", quantize_affine);
    m.impl("dequantize_affine", dequantize_affine);
}

}  // namespace
}  // namespace tpq_gfx950
}  // namespace tensorplay
