// Entry points of the integer matrix product (_int_mm) and of the fused
// int8 GEMM + dequant; the matrix-core kernel itself lives in
// int8_gemm_kernel.h, shared with the ternary matmul.
#include <cstdlib>
#include <type_traits>

#include "int8_decode_kernel.h"
#include "gemm_stagger.h"

namespace tpq {
namespace {

// Which tiled kernel runs a shape.  Three forms, compared by an estimate of their clocks fitted to measurements with the
// weight streaming from HBM (65 .. 2048 rows, K = 2048 .. 11008, N = 2048 .. 11008; the estimate picks the measured
// best or a tie everywhere):
//   tall    256 x 128 tiles, staggered kernel: rounds of 256 tiles x (1,080 clocks per stage of 128 k + 9,000)
//   short   128 x 128 tiles, staggered kernel: its stages are bound by the loads, 690 clocks each, + 8,000
//   both    not below 128 K / 12.5 clocks: a workgroup streams its 128 K bytes of weight at about 25 GB/s per compute
//           unit from HBM, whatever the depth of its ring (4096 x 4096 on short tiles: 21.5 us at any row count,
//           13 .. 19 us with the weight in the caches)
//   sliced  the k range of the tall tiles cut into slices (lock-step kernel, exact int32 partial sums in a workspace:
//           1,450 clocks per stage, up to 2,000 with 32 and more stages per workgroup) + the pass that adds them, whose
//           traffic (2 x slices x M N x 4 bytes at about 2,500 bytes per clock) is what it costs; only where the caller
//           brings a workspace.
// us, weights rotating through HBM, slices wherever they apply / this plan: 4096 x 4096 at 128 / 512 / 1024 rows 17.2 /
// 25.1 / 32.8 -> 17.2 / 21.3 / 22.4; 4096 -> 11008 at 65 / 256 rows 23.9 / 29.3 -> 21.6 / 24.2; 8192 x 8192 at 384 / 512
// rows 49.0 / 52.1 -> 43.4 / 43.3; 11008 -> 4096 at 1024 rows 63.3 -> 57.1; 2048 x 2048 at 512 / 1024 rows 15.1 / 19.9 ->
// 12.6 / 12.5.
// Measured against the lock-step kernel with the same result bits (us, lock-step / staggered tall): 2048 x 4096 x 4096
// 35.9 / 29.0, 2048 x 11008 x 4096 105 / 93, 2048 x 4096 x 11008 91 / 72, 8192^3 550 / 437, 2048 x 2560 x 6912 44.5 /
// 35.0, 4096 x 4096 x 512 18.0 / 16.2.  Slices on the staggered kernel gain nothing (few stages per workgroup).
// TPQ_INT8_FORM = dma / stagger / half and TPQ_INT8_PLAN = o (slices wherever they apply) / h in a tuning build force a form.
enum TiledForm { kTall = 0, kShort = 1, kSliced = 2 };
struct TiledPlan {
    TiledForm form;
    int slices;
};
inline TiledPlan plan_tiled(int64_t M, int64_t N, int64_t K, bool may_slice) {
    const double nk = static_cast<double>(K / kDmaRowBytes);
    const int64_t cols = (N + 127) / 128, t256 = ((M + 255) / 256) * cols, t128 = ((M + 127) / 128) * cols;
    const double stream = 128.0 * static_cast<double>(K) / 12.5;  // a tile's weight bytes at what one compute unit pulls from HBM
    const double tall_tile = nk * 1080.0 + 9000.0, short_tile = nk * 690.0 + 8000.0;
    const double tall = static_cast<double>((t256 + 255) / 256) * (tall_tile > stream ? tall_tile : stream);
    const double shrt = static_cast<double>((t128 + 255) / 256) * (short_tile > stream ? short_tile : stream);
    double sliced = 1e30;
    const int slices = may_slice ? dma_slices(M, N, K) : 1;
    if (slices >= 2) {
        const double per = static_cast<double>((K / kDmaRowBytes + slices - 1) / slices);
        const double stage = 1450.0 + 550.0 * (per < 32.0 ? per / 32.0 : 1.0);
        sliced = per * stage + 9000.0 + 3200.0 + 2.0 * static_cast<double>(M) * static_cast<double>(N) * 4.0 * slices / 2500.0;
    }
    const char* env = tuning_env("TPQ_INT8_PLAN");  // o: slices wherever they apply, else tall; h: short
    if (K >= (1 << 23) || (env && env[0] == 'o')) return TiledPlan{slices >= 2 ? kSliced : kTall, slices >= 2 ? slices : 1};  // K: beyond the staggered kernel's offsets
    if (env && env[0] == 'h') return TiledPlan{kShort, 1};
    // One round of short tiles is never slower than the tall ones on the same problem (fewer compute units busy on tall
    // tiles, and those run at the power limit: 768 rows of 11008 -> 4096 from HBM 55 us short, 81 tall).
    const bool one_round_short = t128 <= 256;
    const double unsliced = one_round_short ? shrt : (shrt < tall ? shrt : tall);
    if (sliced < unsliced) return TiledPlan{kSliced, slices};
    return TiledPlan{one_round_short || shrt < tall ? kShort : kTall, 1};
}

template <class Tile>
int launch_tiled(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Tile tile, hipStream_t s, int slices = 1) {
    const char* env = tuning_env("TPQ_INT8_FORM");
    if (slices > 1) {
        if (env && env[0] == 's') return launch_stagger(a, w, M, N, K, tile, s, slices);
        // up to 128 rows the 256-row tiles of the lock-step kernel are half empty: the 128-row staggered tiles, cut the
        // same way (us, 33 / 128 rows: 4096 x 4096 14.2 / 15.7 -> 12.2 / 14.5, 11008 -> 4096 21.3 / 23.6 -> 18.1 / 21.5,
        // 8192 x 8192 26.2 / 29.5 -> 22.3 / 26.9)
        if ((env && env[0] == 'h') || (!env && M <= 128 && K < (1 << 23)))
            return launch_stagger_bytes<ArithI8, 2>(a, w, M, N, K, tile, s, slices, "int8 mfma gemm (staggered, 128 rows, slices)");
        return launch_dma(a, w, M, N, K, tile, s, slices);
    }
    if (K >= (1 << 23) || (env && env[0] == 'd')) return launch_dma(a, w, M, N, K, tile, s, 1);
    const bool use_short = env ? env[0] == 'h' : plan_tiled(M, N, K, false).form == kShort;
    if (use_short) return launch_stagger_bytes<ArithI8, 2>(a, w, M, N, K, tile, s, 1, "int8 mfma gemm (staggered, 128 rows)");
    return launch_stagger(a, w, M, N, K, tile, s, 1);
}

// partial [slices][M][N] int32 (16-byte aligned) := the slices of A W^T
inline int launch_tiled_sliced(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, int32_t* partial, int slices, hipStream_t s) {
    const TileInt32 tile{partial, nullptr, nullptr, nullptr};
    return launch_tiled(a, w, M, N, K, tile, s, slices);
}

// Large problems with K a multiple of the 128-byte stage take the ring-buffered kernel.
inline TileInt32 to_tile(const EpilogueInt32& ep) { return TileInt32{ep.c, nullptr, nullptr, nullptr}; }
template <int DT>
TileDequant<DT> to_tile(const EpilogueDequant<DT>& ep) {
    return TileDequant<DT>{ep.out, ep.rs, ep.cs, ep.bias};
}

// the epilogue of a slab of rows starting at m0: same operation, pointers moved to that row
inline EpilogueInt32 rebase_rows(const EpilogueInt32& ep, int64_t m0, int64_t N) { return EpilogueInt32{ep.c + m0 * N}; }
template <int DT>
EpilogueDequant<DT> rebase_rows(const EpilogueDequant<DT>& ep, int64_t m0, int64_t N) {
    return EpilogueDequant<DT>{ep.out + m0 * N, ep.rs + m0, ep.cs, ep.bias};
}

// Up to this many rows the decode kernel streams the weight once per 32 rows.
inline int int8_decode_rows(int64_t N) {
    static const int forced = [] { const char* e = tuning_env("TPQ_INT8_DECODE_ROWS"); return e ? std::atoi(e) : -1; }();
    return forced >= 0 ? forced : (N >= 10240 ? 32 : 64);
}

// Slices of the k range the tiled kernel would be cut into for this shape (1: not cut); see dma_slices.
// With a workspace at hand the decode kernel keeps only what it does in one pass (32 rows): two passes cost more
// than the sliced kernel (K = N = 8192, 48 rows: 41 us against 28).
inline int int8_slices(const void* a, const void* w, int64_t M, int64_t N, int64_t K) {
    const char* force = tuning_env("TPQ_INT8_KERNEL");
    if (K <= 0 || !mfma_path_ok(a, w, M, N, K) || (force && force[0] == 'r')) return 1;
    const int decode_rows = int8_decode_rows(N) < 32 ? int8_decode_rows(N) : 32;
    if (M <= decode_rows && int8_decode_ok(a, w, M, N, K)) return 1;
    const TiledPlan plan = plan_tiled(M, N, K, true);
    return plan.form == kSliced ? plan.slices : 1;
}

// partial [slices][M][N] int32 -> out: acc = sum of the slices (exact), then (float(acc) * rs[m]) * cs[n] (+ bias[n]),
// the arithmetic of the fused epilogues
template <int DT>
__global__ __launch_bounds__(256) void int8_finish_kernel(const int32_t* __restrict__ partial, int slices, const float* __restrict__ rs,
                                                          const float* __restrict__ cs, const float* __restrict__ bias,
                                                          typename Elem<DT>::storage* __restrict__ out, int64_t M, int64_t N) {
    const int64_t total = M * N, stride = static_cast<int64_t>(gridDim.x) * 256;
    const bool has_bias = bias != nullptr;
    if (N % 4 == 0) {  // four consecutive columns of one row per thread; grid.y walks the rows, so nothing is divided
        const bool vector_out = (reinterpret_cast<uintptr_t>(out) & (4 * sizeof(typename Elem<DT>::storage) - 1)) == 0;
        for (int64_t m = blockIdx.y; m < M; m += gridDim.y) {
            for (int64_t n = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4; n < N; n += stride * 4) {
                const int64_t idx = m * N + n;
                // the scales first: they are not behind the partial sums when those arrive
                const float4 c = *reinterpret_cast<const float4*>(cs + n);
                const float4 b = has_bias ? *reinterpret_cast<const float4*>(bias + n) : make_float4(0, 0, 0, 0);
                const float r = rs[m];
                int4 v = make_int4(0, 0, 0, 0);
                // four slices requested together (a loop of load and add would wait for memory once per slice); a
                // batch past the last slice asks for the last one again and leaves it out of the sum
                for (int z0 = 0; z0 < slices; z0 += 4) {
                    uint4 p[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) p[j] = nt_load(reinterpret_cast<const uint4*>(partial + (z0 + j < slices ? z0 + j : slices - 1) * total + idx));
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (z0 + j < slices) {
                            v.x += static_cast<int>(p[j].x); v.y += static_cast<int>(p[j].y); v.z += static_cast<int>(p[j].z); v.w += static_cast<int>(p[j].w);
                        }
                }
                const typename Elem<DT>::storage o[4] = {TileDequant<DT>::convert(v.x, r, c.x, b.x, has_bias), TileDequant<DT>::convert(v.y, r, c.y, b.y, has_bias),
                                                        TileDequant<DT>::convert(v.z, r, c.z, b.z, has_bias), TileDequant<DT>::convert(v.w, r, c.w, b.w, has_bias)};
                if (vector_out) {
                    if constexpr (sizeof(typename Elem<DT>::storage) == 2) {
                        *reinterpret_cast<uint2*>(out + idx) = make_uint2(static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16),
                                                                          static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16));
                    } else {
                        *reinterpret_cast<float4*>(out + idx) = make_float4(o[0], o[1], o[2], o[3]);
                    }
                } else {
                    out[idx] = o[0]; out[idx + 1] = o[1]; out[idx + 2] = o[2]; out[idx + 3] = o[3];
                }
            }
        }
        return;
    }
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; idx < total; idx += stride) {
        const int64_t m = idx / N, n = idx - m * N;
        int acc = 0;
        for (int z = 0; z < slices; ++z) acc += partial[z * total + idx];
        out[idx] = TileDequant<DT>::convert(acc, rs[m], cs[n], has_bias ? bias[n] : 0.0f, has_bias);
    }
}

// c [M][N] = sum of the slices (exact)
__global__ __launch_bounds__(256) void int32_sum_slices_kernel(const int32_t* __restrict__ partial, int slices, int32_t* __restrict__ c, int64_t total) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t q = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; q < total / 4; q += stride) {  // total % 4 == 0
        int4 v = make_int4(0, 0, 0, 0);
        for (int z = 0; z < slices; ++z) {
            const uint4 p = nt_load(reinterpret_cast<const uint4*>(partial + z * total) + q);
            v.x += static_cast<int>(p.x); v.y += static_cast<int>(p.y); v.z += static_cast<int>(p.z); v.w += static_cast<int>(p.w);
        }
        reinterpret_cast<int4*>(c)[q] = v;
    }
}

template <class Epilogue>
int launch_best(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Epilogue ep, hipStream_t s) {
    const char* force = tuning_env("TPQ_INT8_KERNEL");  // "reg" keeps the register-staged kernel
    // a few rows: stream the weight once per 32 rows through the decode kernel.  K = N = 4096: 16 rows 6.9 us,
    // 32 rows 9.1 us, 64 rows 17.8 us, against 27.5 us for the tiled kernels below at any of these row counts
    // (28672 -> 8192: 61 / 69 / 138 us against 182 us; 4096 -> 11008: 15 / 21 / 41 us against 31 / 31 / 32 us)
    // Wide N gives the tiled kernel enough tiles earlier (8192 -> 28672: 99 us at 65 rows against 133 at 48).
    const int decode_rows = int8_decode_rows(N);
    if (M <= decode_rows && int8_decode_ok(a, w, M, N, K) && !(force && force[0] == 'r'))
        return launch_int8_decode(a, w, M, N, K, ep, [N](const Epilogue& e, int64_t m0) { return rebase_rows(e, m0, N); }, s);
    // The ring-buffered kernel also wins when its 256 x 128 tiles fill only part of the chip: at K = N = 4096,
    // M = 512 / 1024 it takes 27.9 / 29.5 us against 33.9 / 39.4 us for the register-staged kernel on 128 x 64 tiles.
    // (65 .. 128 rows included: on 128 x 128 tiles 128 rows of 4096 x 4096 take 15 us, 24.6 on the register-staged kernel)
    if (K % kDmaRowBytes == 0 && !(force && force[0] == 'r')) return launch_tiled(a, w, M, N, K, to_tile(ep), s);
    return launch_mfma(a, w, M, N, K, ep, s);
}

// Any strides, any K, signed or unsigned left operand: 16x16 outputs per
// workgroup, operands staged through LDS 16 k at a time.
template <typename LhsT, class Epilogue>
__global__ __launch_bounds__(256) void int_mm_generic_kernel(const LhsT* __restrict__ a,
                                                             const int8_t* __restrict__ b,
                                                             int64_t sbk, int64_t sbn, int64_t M,
                                                             int64_t K, int64_t N, Epilogue ep) {
    __shared__ int sa[16][17], sb[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int64_t m = blockIdx.y * 16ll + ty, n = blockIdx.x * 16ll + tx;
    int acc = 0;
    for (int64_t k0 = 0; k0 < K; k0 += 16) {
        const int64_t ka = k0 + tx, kb = k0 + ty;
        sa[ty][tx] = (m < M && ka < K) ? static_cast<int>(a[m * K + ka]) : 0;
        sb[ty][tx] = (n < N && kb < K) ? static_cast<int>(b[kb * sbk + n * sbn]) : 0;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; ++k) acc += sa[ty][k] * sb[k][tx];
        __syncthreads();
    }
    if (m < M && n < N) ep.store(m * N + n, static_cast<int>(m), static_cast<int>(n), acc);
}

__global__ __launch_bounds__(256) void fill_zero_i32(int32_t* p, int64_t n) {
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += gridDim.x * 256ll) p[i] = 0;
}

template <class Epilogue>
int launch_generic(const void* a, int a_unsigned, const int8_t* b, int64_t sbk, int64_t sbn,
                   int64_t M, int64_t K, int64_t N, Epilogue ep, hipStream_t s) {
    const int64_t gx = (N + 15) / 16, gy = (M + 15) / 16;
    TPQ_REQUIRE(gx <= 0x7FFFFFFF && gy <= 65535, TPQ_ERR_INVALID_VALUE, "_int_mm: shape too large for the generic path");
    const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy));
    if (a_unsigned)
        int_mm_generic_kernel<uint8_t, Epilogue><<<grid, 256, 0, s>>>(static_cast<const uint8_t*>(a), b, sbk, sbn, M, K, N, ep);
    else
        int_mm_generic_kernel<int8_t, Epilogue><<<grid, 256, 0, s>>>(static_cast<const int8_t*>(a), b, sbk, sbn, M, K, N, ep);
    return check_launch("_int_mm generic");
}

// Scratch of the allocation-free entry point: one copy per GPU, held until the process ends.
constexpr int64_t kNoAllocScratchBytes = int64_t{16} << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

// Device address of this GPU's copy of `scratch`.  In host code the array's name is only a handle for
// hipGetSymbolAddress: each GPU has its own copy at its own address, looked up once per device.
int noalloc_scratch(void** out) {
    constexpr int kMaxDevices = 64;
    static std::atomic<void*> per_device[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(TPQ_ERR_RUNTIME, "int8_mm_dequant_noalloc: no current device");
    TPQ_REQUIRE(dev >= 0 && dev < kMaxDevices, TPQ_ERR_RUNTIME, "int8_mm_dequant_noalloc: device id %d out of range", dev);
    void* p = per_device[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr)
            return fail(TPQ_ERR_RUNTIME, "int8_mm_dequant_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
        per_device[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return TPQ_OK;
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int tpq_int_mm(const void* a, int a_unsigned, const int8_t* b, int64_t b_stride_k,
                          int64_t b_stride_n, int32_t* c, int64_t M, int64_t K, int64_t N,
                          void* stream) {
    TPQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "_int_mm: negative shape");
    if (M == 0 || N == 0) return TPQ_OK;
    TPQ_REQUIRE(c, TPQ_ERR_INVALID_VALUE, "_int_mm: null destination");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (K == 0) {  // empty reduction: zeros (p10/src/backend/cuda/IntMM.cu:388-394)
        const int64_t total = M * N;
        const int64_t blocks = (total + 255) / 256;
        fill_zero_i32<<<static_cast<unsigned>(blocks > 8192 ? 8192 : blocks), 256, 0, s>>>(c, total);
        return check_launch("_int_mm zero fill");
    }
    TPQ_REQUIRE(a && b, TPQ_ERR_INVALID_VALUE, "_int_mm: null operand");
    const EpilogueInt32 ep{c};
    if (!a_unsigned && b_stride_k == 1 && b_stride_n == K && mfma_path_ok(a, b, M, N, K))
        return launch_best(static_cast<const int8_t*>(a), b, M, N, K, ep, s);
    return launch_generic(a, a_unsigned, b, b_stride_k, b_stride_n, M, K, N, ep, s);
}

TPQ_EXPORT int tpq_int8_mm_dequant(const int8_t* a, const int8_t* w, const float* row_scale,
                                   const float* col_scale, const float* bias, void* out,
                                   int out_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
    TPQ_REQUIRE(M >= 0 && N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "int8_mm_dequant: negative shape");
    TPQ_REQUIRE(out_dtype == TPQ_DTYPE_F32 || out_dtype == TPQ_DTYPE_F16 || out_dtype == TPQ_DTYPE_BF16,
                TPQ_ERR_INVALID_TYPE, "int8_mm_dequant: unsupported output dtype");
    if (M == 0 || N == 0) return TPQ_OK;
    TPQ_REQUIRE(out && row_scale && col_scale && (K == 0 || (a && w)), TPQ_ERR_INVALID_VALUE,
                "int8_mm_dequant: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool fast = K > 0 && mfma_path_ok(a, w, M, N, K);
#define TPQ_DISPATCH(DT)                                                                            \
    {                                                                                               \
        const EpilogueDequant<DT> ep{static_cast<typename Elem<DT>::storage*>(out), row_scale,      \
                                     col_scale, bias};                                              \
        if (fast) return launch_best(a, w, M, N, K, ep, s);                                         \
        return launch_generic(a, 0, w, 1, K, M, K, N, ep, s);                                       \
    }
    switch (out_dtype) {
        case TPQ_DTYPE_F32: TPQ_DISPATCH(TPQ_DTYPE_F32)
        case TPQ_DTYPE_F16: TPQ_DISPATCH(TPQ_DTYPE_F16)
        default: TPQ_DISPATCH(TPQ_DTYPE_BF16)
    }
#undef TPQ_DISPATCH
}

TPQ_EXPORT int64_t tpq_int8_mm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    // operand alignment is checked again at the call; a 16-byte aligned pair stands in for it here
    const int slices = int8_slices(reinterpret_cast<const void*>(16), reinterpret_cast<const void*>(16), M, N, K);
    return slices >= 2 ? slices * M * N * 4 : 0;
}

TPQ_EXPORT int tpq_int8_mm_dequant_ws(const int8_t* a, const int8_t* w, const float* row_scale, const float* col_scale,
                                      const float* bias, void* out, int out_dtype, int64_t M, int64_t N, int64_t K,
                                      void* workspace, int64_t workspace_bytes, void* stream) {
    const int slices = (M > 0 && N > 0 && K > 0 && a && w) ? int8_slices(a, w, M, N, K) : 1;
    if (slices < 2 || workspace == nullptr || workspace_bytes < slices * M * N * 4 || !aligned(workspace, 16) || (M * N) % 4 != 0 ||
        !aligned(col_scale, 16) || !aligned(bias, 16))
        return tpq_int8_mm_dequant(a, w, row_scale, col_scale, bias, out, out_dtype, M, N, K, stream);
    TPQ_REQUIRE(out_dtype == TPQ_DTYPE_F32 || out_dtype == TPQ_DTYPE_F16 || out_dtype == TPQ_DTYPE_BF16,
                TPQ_ERR_INVALID_TYPE, "int8_mm_dequant: unsupported output dtype");
    TPQ_REQUIRE(out && row_scale && col_scale, TPQ_ERR_INVALID_VALUE, "int8_mm_dequant: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    int32_t* acc = static_cast<int32_t*>(workspace);  // [slices][M][N]; M N % 4 == 0 keeps every matrix 16-byte aligned
    if (int rc = launch_tiled_sliced(a, w, M, N, K, acc, slices, s)) return rc;
    // N % 4 == 0: grid.x over the row's groups of four columns, grid.y over the rows; else a flat grid
    const int64_t items = N % 4 == 0 ? N / 4 : M * N;
    const int64_t blocks = (items + 255) / 256;
    const dim3 grid(static_cast<unsigned>(blocks > 4096 ? 4096 : blocks), N % 4 == 0 ? static_cast<unsigned>(M > 65535 ? 65535 : M) : 1u);
    switch (out_dtype) {
        case TPQ_DTYPE_F32: int8_finish_kernel<TPQ_DTYPE_F32><<<grid, 256, 0, s>>>(acc, slices, row_scale, col_scale, bias, static_cast<float*>(out), M, N); break;
        case TPQ_DTYPE_F16: int8_finish_kernel<TPQ_DTYPE_F16><<<grid, 256, 0, s>>>(acc, slices, row_scale, col_scale, bias, static_cast<uint16_t*>(out), M, N); break;
        default: int8_finish_kernel<TPQ_DTYPE_BF16><<<grid, 256, 0, s>>>(acc, slices, row_scale, col_scale, bias, static_cast<uint16_t*>(out), M, N); break;
    }
    return check_launch("int8_mm_dequant (finish)");
}

TPQ_EXPORT int tpq_int_mm_ws(const void* a, int a_unsigned, const int8_t* b, int64_t b_stride_k, int64_t b_stride_n, int32_t* c,
                             int64_t M, int64_t K, int64_t N, void* workspace, int64_t workspace_bytes, void* stream) {
    const bool sliceable = M > 0 && N > 0 && K > 0 && a && b && c && !a_unsigned && b_stride_k == 1 && b_stride_n == K;
    const int slices = sliceable ? int8_slices(a, b, M, N, K) : 1;
    if (slices < 2 || workspace == nullptr || workspace_bytes < slices * M * N * 4 || !aligned(workspace, 16) || (M * N) % 4 != 0 ||
        !aligned(c, 16))
        return tpq_int_mm(a, a_unsigned, b, b_stride_k, b_stride_n, c, M, K, N, stream);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int32_t* partial = static_cast<int32_t*>(workspace);
    if (int rc = launch_tiled_sliced(static_cast<const int8_t*>(a), b, M, N, K, partial, slices, s)) return rc;
    const int64_t blocks = (M * N / 4 + 255) / 256;
    int32_sum_slices_kernel<<<static_cast<unsigned>(blocks > 4096 ? 4096 : blocks), 256, 0, s>>>(partial, slices, c, M * N);
    return check_launch("_int_mm (sum of slices)");
}

TPQ_EXPORT int64_t tpq_int8_mm_noalloc_max_bytes(void) { return kNoAllocScratchBytes; }

TPQ_EXPORT int tpq_int8_mm_dequant_noalloc(const int8_t* a, const int8_t* w, const float* row_scale, const float* col_scale,
                                           const float* bias, void* out, int out_dtype, int64_t M, int64_t N, int64_t K,
                                           void* stream) {
    const int64_t need = tpq_int8_mm_workspace_bytes(M, N, K);
    TPQ_REQUIRE(need <= kNoAllocScratchBytes, TPQ_ERR_INVALID_VALUE,
                "int8_mm_dequant_noalloc: %lld x %lld x %lld needs %lld bytes of scratch, the built-in buffer holds %lld",
                static_cast<long long>(M), static_cast<long long>(N), static_cast<long long>(K), static_cast<long long>(need),
                static_cast<long long>(kNoAllocScratchBytes));
    if (need == 0) return tpq_int8_mm_dequant(a, w, row_scale, col_scale, bias, out, out_dtype, M, N, K, stream);
    void* ws = nullptr;
    if (int rc = noalloc_scratch(&ws)) return rc;
    // every slice matrix is written in full before the finishing kernel reads it: nothing to clear between calls
    return tpq_int8_mm_dequant_ws(a, w, row_scale, col_scale, bias, out, out_dtype, M, N, K, ws, kNoAllocScratchBytes, stream);
}
