// Error state, ABI version, and the small memory-bound kernels of the path:
// the stand-alone rescale and the weight packers.
#include "tpq_common.h"

namespace tpq {

char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

namespace {

// ---------------------------------------------------------------------------
// out = (float(acc) * rs[m]) * cs[n]; four columns per lane when N % 4 == 0.
// Multiplication order follows the reference's kernels
// (p10/include/QuantNativeImpl.h:1258-1259,
//  p10/src/backend/cuda/QuantGemmKernels.cu:1619-1621).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rescale_vec4(const int4* __restrict__ acc,
                                                    const float* __restrict__ rs,
                                                    const float4* __restrict__ cs,
                                                    float4* __restrict__ out, int64_t M, int N4) {
    const int64_t total = M * N4;
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < total; i += gridDim.x * 256ll) {
        const int64_t m = i / N4;
        const int n4 = static_cast<int>(i - m * N4);
        const int4 a = acc[i];
        const float r = rs[m];
        const float4 c = cs[n4];
        float4 o;
        o.x = __fmul_rn(__fmul_rn(static_cast<float>(a.x), r), c.x);
        o.y = __fmul_rn(__fmul_rn(static_cast<float>(a.y), r), c.y);
        o.z = __fmul_rn(__fmul_rn(static_cast<float>(a.z), r), c.z);
        o.w = __fmul_rn(__fmul_rn(static_cast<float>(a.w), r), c.w);
        out[i] = o;
    }
}

__global__ __launch_bounds__(256) void rescale_scalar(const int32_t* __restrict__ acc,
                                                      const float* __restrict__ rs,
                                                      const float* __restrict__ cs,
                                                      float* __restrict__ out, int64_t M, int64_t N) {
    const int64_t total = M * N;
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < total; i += gridDim.x * 256ll) {
        const int64_t m = i / N;
        out[i] = __fmul_rn(__fmul_rn(static_cast<float>(acc[i]), rs[m]), cs[i - m * N]);
    }
}

// ---------------------------------------------------------------------------
// int4 weight pack into the device layout.  One lane per output word:
//   word(nT, kO, t, i2): n = 8 nT + t/4, k0 = (kO*I + 2 i2)*16 + 2 (t%4)
//   bits[4j .. 4j+3]     = code[n, k0 + 8j]       j = 0..3
//   bits[16+4j .. 19+4j] = code[n, k0 + 8j + 1]
// which is what the reference's two kernels (nibble pack with even k in the
// high nibble, then the fragment shuffle) produce together
// (p10/src/backend/cuda/QuantGemmKernels.cu:322-330, 838-877); codes outside
// [N,K] contribute zero nibbles.  Adjacent lanes read adjacent code pairs, so
// a wavefront reads 8 rows x 8 bytes per j: sector-sized pieces of the int32
// code matrix, each touched once.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void int4_pack_words(const int32_t* __restrict__ codes,
                                                       int32_t* __restrict__ out, int64_t N,
                                                       int64_t K, int inner, int64_t k_super,
                                                       int64_t total_words) {
    const int half_inner = inner >> 1;
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total_words;
         idx += gridDim.x * 256ll) {
        const int i2 = static_cast<int>(idx % half_inner);
        const int64_t rest = idx / half_inner;
        const int t = static_cast<int>(rest & 31);
        const int64_t tile = rest >> 5;
        const int64_t kO = tile % k_super;
        const int64_t nT = tile / k_super;
        const int64_t n = nT * 8 + (t >> 2);
        const int64_t k0 = (kO * inner + 2 * i2) * 16 + 2 * (t & 3);
        uint32_t word = 0;
        if (n < N) {
            const int32_t* row = codes + n * K;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int64_t k = k0 + 8 * j;
                // K is even and k is even, so the pair is inside or outside together
                if (k < K) {
                    const int2 pair = *reinterpret_cast<const int2*>(row + k);
                    word |= (static_cast<uint32_t>(pair.x) & 15u) << (4 * j);
                    word |= (static_cast<uint32_t>(pair.y) & 15u) << (16 + 4 * j);
                }
            }
        }
        out[idx] = static_cast<int32_t>(word);
    }
}

// ---------------------------------------------------------------------------
// Ternary pack / unpack (tensorplay/ao/quantization/bitnet.py:72-107).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ternary_pack_bytes(const int8_t* __restrict__ codes,
                                                          uint8_t* __restrict__ out, int64_t rows,
                                                          int64_t cols, int64_t bytes_per_row) {
    const int64_t total = rows * bytes_per_row;
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < total; i += gridDim.x * 256ll) {
        const int64_t r = i / bytes_per_row;
        const int64_t k = (i - r * bytes_per_row) * 4;
        const int8_t* src = codes + r * cols + k;
        uint32_t v = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int c = (k + q < cols) ? src[q] : 0;
            v |= (static_cast<uint32_t>(c) & 3u) << (6 - 2 * q);
        }
        out[i] = static_cast<uint8_t>(v);
    }
}

__global__ __launch_bounds__(256) void ternary_unpack_bytes(const uint8_t* __restrict__ packed,
                                                            int8_t* __restrict__ out, int64_t rows,
                                                            int64_t cols, int64_t bytes_per_row) {
    const int64_t total = rows * bytes_per_row;
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < total; i += gridDim.x * 256ll) {
        const int64_t r = i / bytes_per_row;
        const int64_t k = (i - r * bytes_per_row) * 4;
        const uint32_t b = static_cast<uint32_t>(packed[i]) << 24;  // byte in the top of the word
        int8_t* dst = out + r * cols + k;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (k + q < cols)  // arithmetic shift sign-extends the 2-bit field
                dst[q] = static_cast<int8_t>(static_cast<int32_t>(b << (2 * q)) >> 30);
    }
}

inline unsigned grid_for(int64_t items, int per_block = 256, unsigned cap = 256u * 32u) {
    const int64_t blocks = (items + per_block - 1) / per_block;
    return static_cast<unsigned>(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}


// ---------------------------------------------------------------------------
// int4 CPU layout (p10/src/backend/cpu/QuantizedElementwiseKernels.cpp:370-390): uint8 [N, K/2];
// N in blocks of `columns`; inside a block, for each k, width/2 bytes; byte `lane` of a full block
// on a vector tier pairs column lane (low nibble) with lane + width/2 (high nibble), tail blocks and
// the plain tier pair 2*lane with 2*lane + 1.
// ---------------------------------------------------------------------------
struct CpuLayout {
    int64_t N, K;
    int columns, half_split;
    // where code (col, feature) lives: byte index and shift
    __device__ __forceinline__ void locate(int64_t col, int64_t feature, int64_t* byte, int* shift) const {
        const int64_t first = col / columns * columns;
        const int64_t width = N - first < columns ? N - first : columns;
        const int64_t c = col - first;
        const bool full = half_split && width == columns;
        const int64_t lane = full ? c % (width / 2) : c / 2;
        *shift = full ? (c >= width / 2 ? 4 : 0) : static_cast<int>(c & 1) * 4;
        *byte = first * K / 2 + feature * (width / 2) + lane;
    }
};

__global__ __launch_bounds__(256) void int4_pack_cpu_bytes(const int32_t* __restrict__ codes, uint8_t* __restrict__ out,
                                                           CpuLayout lay, int64_t total_bytes) {
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total_bytes; idx += gridDim.x * 256ll) {
        // invert locate(): idx -> (block, feature, lane)
        const int64_t per_block = static_cast<int64_t>(lay.columns) * lay.K / 2;
        const int64_t block = idx / per_block, first = block * lay.columns;
        const int64_t width = lay.N - first < lay.columns ? lay.N - first : lay.columns;
        const int64_t off = idx - first * lay.K / 2;
        const int64_t feature = off / (width / 2), lane = off % (width / 2);
        const bool full = lay.half_split && width == lay.columns;
        const int64_t lo = full ? lane : 2 * lane, hi = full ? lane + width / 2 : 2 * lane + 1;
        const uint32_t a = static_cast<uint32_t>(codes[(first + lo) * lay.K + feature]) & 0xFFu;
        const uint32_t b = static_cast<uint32_t>(codes[(first + hi) * lay.K + feature]) & 0xFFu;
        out[idx] = static_cast<uint8_t>(a | (b << 4));
    }
}

// CPU layout -> device layout (innerKTiles = 2): same word indexing as int4_pack_words.
__global__ __launch_bounds__(256) void int4_cpu_to_device_words(const uint8_t* __restrict__ packed, int32_t* __restrict__ out,
                                                                CpuLayout lay, int64_t k_super, int64_t total_words) {
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total_words; idx += gridDim.x * 256ll) {
        const int t = static_cast<int>(idx & 31);
        const int64_t tile = idx >> 5;
        const int64_t kT = tile % k_super, nT = tile / k_super;
        const int64_t n = nT * 8 + (t >> 2);
        const int64_t k0 = kT * 32 + 2 * (t & 3);
        uint32_t word = 0;
        if (n < lay.N) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int odd = 0; odd < 2; ++odd) {
                    const int64_t k = k0 + 8 * j + odd;
                    if (k < lay.K) {
                        int64_t byte;
                        int shift;
                        lay.locate(n, k, &byte, &shift);
                        word |= ((static_cast<uint32_t>(packed[byte]) >> shift) & 15u) << (4 * j + 16 * odd);
                    }
                }
        }
        out[idx] = static_cast<int32_t>(word);
    }
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int tpq_abi_version(void) { return 1; }

#ifdef TPQ_TEST_HOOKS
namespace tpq {
std::atomic<int> g_override_int8_row{-1};
std::atomic<int> g_override_lowbit_row{-1};
std::atomic<int> g_override_int4_row{-1};
}  // namespace tpq

TPQ_EXPORT int tpq_set_kernel_override(const char* route, int value) {
    TPQ_REQUIRE(route != nullptr, TPQ_ERR_INVALID_VALUE, "tpq_set_kernel_override: null route name");
    TPQ_REQUIRE(value >= -1 && value <= 1, TPQ_ERR_INVALID_VALUE, "tpq_set_kernel_override: value must be -1, 0 or 1");
    if (std::strcmp(route, "int8_row") == 0) tpq::g_override_int8_row.store(value, std::memory_order_relaxed);
    else if (std::strcmp(route, "lowbit_row") == 0) tpq::g_override_lowbit_row.store(value, std::memory_order_relaxed);
    else if (std::strcmp(route, "int4_row") == 0) tpq::g_override_int4_row.store(value, std::memory_order_relaxed);
    else return tpq::fail(TPQ_ERR_INVALID_VALUE, "tpq_set_kernel_override: unknown route '%s'", route);
    return TPQ_OK;
}
#endif

TPQ_EXPORT const char* tpq_last_error(void) { return error_buffer(); }

TPQ_EXPORT int tpq_int8_mm_rescale(const int32_t* acc, const float* row_scale,
                                   const float* col_scale, float* out, int64_t M, int64_t N,
                                   void* stream) {
    TPQ_REQUIRE(M >= 0 && N >= 0, TPQ_ERR_INVALID_VALUE, "_int8_mm_rescale(): negative shape");
    if (M == 0 || N == 0) return TPQ_OK;
    TPQ_REQUIRE(acc && row_scale && col_scale && out, TPQ_ERR_INVALID_VALUE,
                "_int8_mm_rescale(): null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (N % 4 == 0 && aligned(acc, 16) && aligned(col_scale, 16) && aligned(out, 16)) {
        rescale_vec4<<<grid_for(M * (N / 4)), 256, 0, s>>>(
            reinterpret_cast<const int4*>(acc), row_scale, reinterpret_cast<const float4*>(col_scale),
            reinterpret_cast<float4*>(out), M, static_cast<int>(N / 4));
    } else {
        rescale_scalar<<<grid_for(M * N), 256, 0, s>>>(acc, row_scale, col_scale, out, M, N);
    }
    return check_launch("tpq_int8_mm_rescale");
}

TPQ_EXPORT int tpq_int4_pack(const int32_t* codes, int64_t N, int64_t K, int inner_k_tiles,
                             int32_t* out, void* stream) {
    TPQ_REQUIRE(N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE,
                "_convert_weight_to_int4pack(): expected 2-D codes [N,K]");
    TPQ_REQUIRE(inner_k_tiles == 2 || inner_k_tiles == 4 || inner_k_tiles == 8,
                TPQ_ERR_INVALID_VALUE, "_convert_weight_to_int4pack(): innerKTiles must be 2, 4 or 8");
    TPQ_REQUIRE(K % 2 == 0, TPQ_ERR_INVALID_VALUE, "_convert_weight_to_int4pack(): K must be even");
    if (N == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(codes && out, TPQ_ERR_INVALID_VALUE, "_convert_weight_to_int4pack(): null pointer");
    TPQ_REQUIRE(aligned(codes, 8), TPQ_ERR_INVALID_VALUE,
                "_convert_weight_to_int4pack(): codes must be 8-byte aligned");
    const int64_t n_tiles = (N + 7) / 8;
    const int64_t k_super = (K + inner_k_tiles * 16 - 1) / (inner_k_tiles * 16);
    const int64_t total = n_tiles * k_super * 32 * (inner_k_tiles / 2);
    int4_pack_words<<<grid_for(total), 256, 0, static_cast<hipStream_t>(stream)>>>(
        codes, out, N, K, inner_k_tiles, k_super, total);
    return check_launch("tpq_int4_pack");
}

TPQ_EXPORT int tpq_ternary_pack(const int8_t* codes, int64_t rows, int64_t cols, uint8_t* out,
                                void* stream) {
    TPQ_REQUIRE(rows >= 0 && cols >= 0, TPQ_ERR_INVALID_VALUE, "pack_ternary: negative shape");
    if (rows == 0 || cols == 0) return TPQ_OK;
    TPQ_REQUIRE(codes && out, TPQ_ERR_INVALID_VALUE, "pack_ternary: null pointer");
    const int64_t bpr = (cols + 3) / 4;
    ternary_pack_bytes<<<grid_for(rows * bpr), 256, 0, static_cast<hipStream_t>(stream)>>>(
        codes, out, rows, cols, bpr);
    return check_launch("tpq_ternary_pack");
}

TPQ_EXPORT int tpq_ternary_unpack(const uint8_t* packed, int64_t rows, int64_t cols, int8_t* out,
                                  void* stream) {
    TPQ_REQUIRE(rows >= 0 && cols >= 0, TPQ_ERR_INVALID_VALUE, "unpack_ternary: negative shape");
    if (rows == 0 || cols == 0) return TPQ_OK;
    TPQ_REQUIRE(packed && out, TPQ_ERR_INVALID_VALUE, "unpack_ternary: null pointer");
    const int64_t bpr = (cols + 3) / 4;
    ternary_unpack_bytes<<<grid_for(rows * bpr), 256, 0, static_cast<hipStream_t>(stream)>>>(
        packed, out, rows, cols, bpr);
    return check_launch("tpq_ternary_unpack");
}

TPQ_EXPORT int tpq_int4_pack_cpu_layout(const int32_t* codes, int64_t N, int64_t K, int block_cols,
                                        int half_split, uint8_t* out, void* stream) {
    TPQ_REQUIRE(N >= 0 && K >= 0, TPQ_ERR_INVALID_VALUE, "_convert_weight_to_int4pack_for_cpu(): negative shape");
    TPQ_REQUIRE(N % 16 == 0 && K % 2 == 0, TPQ_ERR_INVALID_VALUE,
                "_convert_weight_to_int4pack_for_cpu(): N must be a multiple of 16 and K even");
    TPQ_REQUIRE(block_cols == 32 || block_cols == 64, TPQ_ERR_INVALID_VALUE,
                "_convert_weight_to_int4pack_for_cpu(): block width must be 32 or 64");
    if (N == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(codes && out, TPQ_ERR_INVALID_VALUE, "_convert_weight_to_int4pack_for_cpu(): null pointer");
    const CpuLayout lay{N, K, block_cols, half_split ? 1 : 0};
    const int64_t total = N * K / 2;
    int4_pack_cpu_bytes<<<grid_for(total), 256, 0, static_cast<hipStream_t>(stream)>>>(codes, out, lay, total);
    return check_launch("tpq_int4_pack_cpu_layout");
}

TPQ_EXPORT int tpq_int4_cpu_layout_to_device(const uint8_t* packed_cpu, int64_t N, int64_t K, int block_cols,
                                             int half_split, int32_t* out, void* stream) {
    TPQ_REQUIRE(N >= 0 && K >= 0 && N % 16 == 0 && K % 2 == 0, TPQ_ERR_INVALID_VALUE,
                "int4 layout conversion: N must be a multiple of 16 and K even");
    TPQ_REQUIRE(block_cols == 32 || block_cols == 64, TPQ_ERR_INVALID_VALUE,
                "int4 layout conversion: block width must be 32 or 64");
    if (N == 0 || K == 0) return TPQ_OK;
    TPQ_REQUIRE(packed_cpu && out, TPQ_ERR_INVALID_VALUE, "int4 layout conversion: null pointer");
    const CpuLayout lay{N, K, block_cols, half_split ? 1 : 0};
    const int64_t k_super = (K + 31) / 32;
    const int64_t total = (N / 8) * k_super * 32;
    int4_cpu_to_device_words<<<grid_for(total), 256, 0, static_cast<hipStream_t>(stream)>>>(packed_cpu, out, lay, k_super, total);
    return check_launch("tpq_int4_cpu_layout_to_device");
}
