// Block-wise affine quantizer / dequantizer for gfx950.
//
// Arithmetic (reference: p10/src/backend/cpu/QuantKernels.cpp:365-455, the device twin is
// p10/src/backend/cuda/AffineQuantKernels.cu:818-901):
//   inv      = scale == 0 ? 1 : 1 / scale                       (IEEE divide)
//   position = rint(x * inv) [+ zero_point]                      (fp32, round half to even)
//   code     = clamp(int64(position), quant_min, quant_max)      (NaN / out of range -> INT64_MIN)
// and for the packed 4/2/1-bit storages the int64 is first cut to its low 32 bits, the clamp is
// done on that int32 and element i goes to bits (i % pack) * bits of byte i / pack.
// Dequantize: x = (float(code) - zero_point) * scale.
//
// Both directions are one pass over HBM (4 bytes + 1 byte or less per element).  The block grid
// of every layout that occurs on the weight / activation path (per tensor, per row, groups
// along the last dimension, per leading channel) collapses to "rows of K contiguous elements
// cut into groups of g".  When K and g are multiples of four, a thread works on pieces of four
// consecutive elements and consecutive lanes on consecutive pieces, so every wavefront load or
// store of the float side is whole cache lines (measured 4.6 TB/s quantizing and 5.1 TB/s
// dequantizing 4096 x 4096 to packed 4-bit; 16 contiguous elements per thread instead gave 4.2 and
// 2.4 TB/s).  Other K / g: a thread takes 16 consecutive elements and walks (row, group) with
// counters.  Any other grid (blocks that tile two dimensions at once) takes the general kernel, one
// thread per output byte with the full index arithmetic.
#include "tpq_common.h"

namespace tpq {
namespace {

constexpr int kChunk = 16;     // elements per thread in the run kernel
constexpr int kMaxDims = 8;

struct Storage {
    int bits;        // 8, 32, 4, 2, 1
    int is_signed;   // int8 / int32
    int64_t lo, hi;  // representable range
};

bool storage_of(int tag, Storage* st) {
    switch (tag) {
        case TPQ_STORAGE_I8: *st = {8, 1, -128, 127}; return true;
        case TPQ_STORAGE_U8: *st = {8, 0, 0, 255}; return true;
        case TPQ_STORAGE_I32: *st = {32, 1, INT32_MIN, INT32_MAX}; return true;
        case TPQ_STORAGE_U4X2: *st = {4, 0, 0, 15}; return true;
        case TPQ_STORAGE_U2X4: *st = {2, 0, 0, 3}; return true;
        case TPQ_STORAGE_U1X8: *st = {1, 0, 0, 1}; return true;
        default: return false;
    }
}

// ---- the block grid -----------------------------------------------------------

struct Grid {
    int dim;
    int64_t sizes[kMaxDims], blocks[kMaxDims], block_stride[kMaxDims], size_stride[kMaxDims];
};

struct Runs {  // rows of K contiguous elements, groups of g along each row, G groups per row
    int64_t K, g, G;
};

struct Plan {
    Grid grid;
    int64_t numel, num_blocks;
    bool as_runs;
    Runs runs;
};

int make_plan(const char* op, int ndim, const int64_t* sizes, const int64_t* block_size, Plan* plan) {
    TPQ_REQUIRE(ndim >= 0 && ndim <= kMaxDims, TPQ_ERR_UNSUPPORTED, "%s: at most %d dimensions are built (got %d)", op, kMaxDims, ndim);
    Grid& gr = plan->grid;
    gr.dim = ndim;
    plan->numel = 1;
    for (int d = 0; d < ndim; ++d) {
        TPQ_REQUIRE(sizes[d] >= 0, TPQ_ERR_INVALID_VALUE, "%s: negative size", op);
        TPQ_REQUIRE(block_size[d] > 0, TPQ_ERR_INVALID_VALUE, "%s: block_size entries must be positive", op);
        plan->numel *= sizes[d];
    }
    int64_t stride = 1, blocks_after = 1;
    plan->num_blocks = 1;
    for (int d = ndim - 1; d >= 0; --d) {
        gr.sizes[d] = sizes[d];
        gr.size_stride[d] = stride;
        stride *= sizes[d];
        const int64_t b = block_size[d] < sizes[d] ? block_size[d] : sizes[d];
        gr.blocks[d] = b > 0 ? b : 1;
        const int64_t per_dim = (sizes[d] + gr.blocks[d] - 1) / gr.blocks[d];
        gr.block_stride[d] = blocks_after;
        blocks_after *= per_dim;
        plan->num_blocks *= per_dim;
    }
    for (int d = ndim; d < kMaxDims; ++d) gr.sizes[d] = gr.blocks[d] = gr.block_stride[d] = gr.size_stride[d] = 1;

    // trailing dimensions that one block covers whole merge into the dimension before them
    int d = ndim - 1;
    int64_t inner = 1;
    while (d >= 0 && gr.blocks[d] == gr.sizes[d]) inner *= gr.sizes[d--];
    plan->as_runs = true;
    if (d < 0) {
        plan->runs = {plan->numel, plan->numel, 1};
    } else {
        for (int e = 0; e < d; ++e) plan->as_runs = plan->as_runs && gr.blocks[e] == 1;
        plan->runs = {gr.sizes[d] * inner, gr.blocks[d] * inner, (gr.sizes[d] + gr.blocks[d] - 1) / gr.blocks[d]};
    }
    return TPQ_OK;
}

__device__ __forceinline__ int64_t block_of(const Grid& gr, int64_t linear) {
    int64_t b = 0;
    for (int d = 0; d < gr.dim; ++d) {
        const int64_t coord = (linear / gr.size_stride[d]) % gr.sizes[d];
        b += (coord / gr.blocks[d]) * gr.block_stride[d];
    }
    return b;
}

// ---- one element ------------------------------------------------------------------

struct Params {
    const float* scales;
    const float* zeros;  // null: no zero point
    int scale_is_scalar, zero_is_scalar;
    int32_t qmin, qmax;
};

__device__ __forceinline__ float inverse_of(float scale) { return scale == 0.0f ? 1.0f : __fdiv_rn(1.0f, scale); }

// SUB = packed 4/2/1-bit storage (int32 wrap before the clamp); otherwise the clamp is on the int64.
template <bool SUB>
__device__ __forceinline__ int32_t quantize_one(float x, float inv, float zero, bool has_zero, int32_t qmin, int32_t qmax) {
    const float r = __builtin_rintf(x * inv);
    const float position = has_zero ? r + zero : r;
    const bool in_range = position >= -0x1p63f && position < 0x1p63f;  // false for NaN
    int32_t q;
    if (__builtin_fabsf(position) < 0x1p31f) {
        q = static_cast<int32_t>(position);
    } else if (SUB) {
        const int64_t wide = in_range ? static_cast<int64_t>(position) : INT64_MIN;
        q = static_cast<int32_t>(static_cast<uint32_t>(wide));
    } else {
        // quant_min / quant_max lie inside int32, so only the side matters
        return in_range && position > 0.0f ? qmax : qmin;
    }
    return q < qmin ? qmin : q > qmax ? qmax : q;
}

__device__ __forceinline__ float dequantize_one(int32_t code, float scale, float zero) {
    return (static_cast<float>(code) - zero) * scale;
}

// ---- 16-element loads and stores ---------------------------------------------------

template <int DT>
__device__ __forceinline__ void load_floats(const void* x, int64_t c0, int n, float v[kChunk]) {
    using S = typename Elem<DT>::storage;
    const S* p = static_cast<const S*>(x) + c0;
    if (n == kChunk) {
        __attribute__((aligned(16))) S raw[kChunk];
        const uint4* src = reinterpret_cast<const uint4*>(p);
#pragma unroll
        for (int e = 0; e < static_cast<int>(kChunk * sizeof(S) / 16); ++e) reinterpret_cast<uint4*>(raw)[e] = src[e];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) v[e] = Elem<DT>::load(raw[e]);
    } else {
#pragma unroll
        for (int e = 0; e < kChunk; ++e) v[e] = e < n ? Elem<DT>::load(p[e]) : 0.0f;
    }
}

// codes q[0..n) -> storage; BITS = 8 (one byte each), 32, or 4 / 2 / 1 (packed, low bits first)
template <int BITS>
__device__ __forceinline__ void store_codes(void* out, int64_t c0, int n, const int32_t q[kChunk]) {
    if constexpr (BITS == 32) {
        int32_t* p = static_cast<int32_t*>(out) + c0;
        if (n == kChunk) {
#pragma unroll
            for (int e = 0; e < 4; ++e) reinterpret_cast<int4*>(p)[e] = make_int4(q[4 * e], q[4 * e + 1], q[4 * e + 2], q[4 * e + 3]);
        } else {
#pragma unroll
            for (int e = 0; e < kChunk; ++e)
                if (e < n) p[e] = q[e];
        }
    } else {
        constexpr int pack = 8 / BITS;             // codes per byte
        constexpr int bytes = kChunk / pack;       // 16, 8, 4, 2
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            const int byte = e / pack, shift = (e % pack) * BITS;
            // as in the reference the code is not masked: the clamp keeps it inside its field
            const uint32_t code = e < n ? (static_cast<uint32_t>(q[e]) & 0xFFu) << shift : 0u;
            w[byte / 4] |= (code & 0xFFu) << (8 * (byte % 4));
        }
        uint8_t* p = static_cast<uint8_t*>(out) + c0 / pack;  // c0 is a multiple of 16
        if (n == kChunk) {
            if constexpr (bytes == 16) *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
            if constexpr (bytes == 8) *reinterpret_cast<uint2*>(p) = make_uint2(w[0], w[1]);
            if constexpr (bytes == 4) *reinterpret_cast<uint32_t*>(p) = w[0];
            if constexpr (bytes == 2) *reinterpret_cast<uint16_t*>(p) = static_cast<uint16_t>(w[0]);
        } else {
            const int live = (n + pack - 1) / pack;
#pragma unroll
            for (int b = 0; b < bytes; ++b)
                if (b < live) p[b] = static_cast<uint8_t>(w[b / 4] >> (8 * (b % 4)));
        }
    }
}

template <int BITS, bool SIGNED>
__device__ __forceinline__ void load_codes(const void* in, int64_t c0, int n, int32_t q[kChunk]) {
    if constexpr (BITS == 32) {
        const int32_t* p = static_cast<const int32_t*>(in) + c0;
        if (n == kChunk) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int4 t = reinterpret_cast<const int4*>(p)[e];
                q[4 * e] = t.x; q[4 * e + 1] = t.y; q[4 * e + 2] = t.z; q[4 * e + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < kChunk; ++e) q[e] = e < n ? p[e] : 0;
        }
    } else {
        constexpr int pack = 8 / BITS;
        constexpr int bytes = kChunk / pack;
        constexpr uint32_t mask = (1u << BITS) - 1u;
        const uint8_t* p = static_cast<const uint8_t*>(in) + c0 / pack;
        uint32_t w[4] = {0, 0, 0, 0};
        if (n == kChunk) {
            if constexpr (bytes == 16) { const uint4 t = *reinterpret_cast<const uint4*>(p); w[0] = t.x; w[1] = t.y; w[2] = t.z; w[3] = t.w; }
            if constexpr (bytes == 8) { const uint2 t = *reinterpret_cast<const uint2*>(p); w[0] = t.x; w[1] = t.y; }
            if constexpr (bytes == 4) w[0] = *reinterpret_cast<const uint32_t*>(p);
            if constexpr (bytes == 2) w[0] = *reinterpret_cast<const uint16_t*>(p);
        } else {
            const int live = (n + pack - 1) / pack;
#pragma unroll
            for (int b = 0; b < bytes; ++b)
                if (b < live) w[b / 4] |= static_cast<uint32_t>(p[b]) << (8 * (b % 4));
        }
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            const int byte = e / pack, shift = (e % pack) * BITS;
            const uint32_t field = ((w[byte / 4] >> (8 * (byte % 4))) >> shift) & mask;
            q[e] = SIGNED ? static_cast<int32_t>(static_cast<int8_t>(field)) : static_cast<int32_t>(field);
        }
    }
}

// ---- kernels ---------------------------------------------------------------------------

// Walks the (row, group) of 16 consecutive elements; fetch(block) is called when the block changes.
struct RunCursor {
    int64_t block;   // row * G + group
    int64_t col;     // position in the row
    int64_t within;  // position in the group
    __device__ __forceinline__ RunCursor(const Runs& r, int64_t c0) {
        const int64_t row = c0 / r.K;
        col = c0 - row * r.K;
        const int64_t grp = col / r.g;
        within = col - grp * r.g;
        block = row * r.G + grp;
    }
    // true when the next element starts a new block
    __device__ __forceinline__ bool step(const Runs& r) {
        ++col; ++within;
        if (col == r.K) { col = 0; within = 0; ++block; return true; }  // next row: its first group follows in memory order
        if (within == r.g) { within = 0; ++block; return true; }
        return false;
    }
};

template <int DT, int BITS>
__global__ __launch_bounds__(256) void quantize_runs_kernel(const void* __restrict__ x, void* __restrict__ out, int64_t numel,
                                                            Runs runs, Params pr) {
    const int64_t chunks = (numel + kChunk - 1) / kChunk;
    for (int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; c < chunks;
         c += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t c0 = c * kChunk;
        const int n = numel - c0 < kChunk ? static_cast<int>(numel - c0) : kChunk;
        float v[kChunk];
        load_floats<DT>(x, c0, n, v);
        RunCursor cur(runs, c0);
        const bool has_zero = pr.zeros != nullptr;
        float inv = inverse_of(pr.scales[pr.scale_is_scalar ? 0 : cur.block]);
        float zero = has_zero ? pr.zeros[pr.zero_is_scalar ? 0 : cur.block] : 0.0f;
        int32_t q[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            q[e] = quantize_one<(BITS < 8)>(v[e], inv, zero, has_zero, pr.qmin, pr.qmax);
            if (cur.step(runs) && e + 1 < n) {
                inv = inverse_of(pr.scales[pr.scale_is_scalar ? 0 : cur.block]);
                if (has_zero) zero = pr.zeros[pr.zero_is_scalar ? 0 : cur.block];
            }
        }
        store_codes<BITS>(out, c0, n, q);
    }
}

template <int BITS, bool SIGNED>
__global__ __launch_bounds__(256) void dequantize_runs_kernel(const void* __restrict__ in, float* __restrict__ out, int64_t numel,
                                                              Runs runs, Params pr) {
    const int64_t chunks = (numel + kChunk - 1) / kChunk;
    for (int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; c < chunks;
         c += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t c0 = c * kChunk;
        const int n = numel - c0 < kChunk ? static_cast<int>(numel - c0) : kChunk;
        int32_t q[kChunk];
        load_codes<BITS, SIGNED>(in, c0, n, q);
        RunCursor cur(runs, c0);
        const bool has_zero = pr.zeros != nullptr;
        float scale = pr.scales[pr.scale_is_scalar ? 0 : cur.block];
        float zero = has_zero ? pr.zeros[pr.zero_is_scalar ? 0 : cur.block] : 0.0f;
        float v[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            v[e] = dequantize_one(q[e], scale, zero);
            if (cur.step(runs) && e + 1 < n) {
                scale = pr.scales[pr.scale_is_scalar ? 0 : cur.block];
                if (has_zero) zero = pr.zeros[pr.zero_is_scalar ? 0 : cur.block];
            }
        }
        float* p = out + c0;
        if (n == kChunk) {
#pragma unroll
            for (int e = 0; e < 4; ++e) reinterpret_cast<float4*>(p)[e] = make_float4(v[4 * e], v[4 * e + 1], v[4 * e + 2], v[4 * e + 3]);
        } else {
#pragma unroll
            for (int e = 0; e < kChunk; ++e)
                if (e < n) p[e] = v[e];
        }
    }
}

// Rows and groups that are multiples of four: a thread takes pieces of four consecutive elements
// (one block each), consecutive lanes take consecutive pieces, so the float side moves as whole
// cache lines per wavefront instruction.  Four pieces per thread are in flight at once.
struct Pieces {
    int64_t K, g, G;
    int k_shift, g_shift;  // log2 when a power of two, else -1
    int small;             // numel < 2^31: 32-bit index arithmetic
    int need_block;        // some parameter differs between blocks
};

__device__ __forceinline__ int64_t piece_block(const Pieces& ps, int64_t c0) {
    if (!ps.need_block) return 0;
    if (ps.small) {
        const uint32_t c = static_cast<uint32_t>(c0), K = static_cast<uint32_t>(ps.K), g = static_cast<uint32_t>(ps.g);
        const uint32_t row = ps.k_shift >= 0 ? c >> ps.k_shift : c / K;
        const uint32_t col = c - row * K;
        const uint32_t grp = ps.g_shift >= 0 ? col >> ps.g_shift : col / g;
        return static_cast<int64_t>(row) * ps.G + grp;
    }
    const int64_t row = ps.k_shift >= 0 ? c0 >> ps.k_shift : c0 / ps.K;
    const int64_t col = c0 - row * ps.K;
    const int64_t grp = ps.g_shift >= 0 ? col >> ps.g_shift : col / ps.g;
    return row * ps.G + grp;
}

// the four codes of piece p (elements 4p .. 4p+3)
template <int BITS, bool SIGNED>
__device__ __forceinline__ void load_piece(const void* in, int64_t p, int32_t q[4]) {
    if constexpr (BITS == 32) {
        const int4 t = static_cast<const int4*>(in)[p];
        q[0] = t.x; q[1] = t.y; q[2] = t.z; q[3] = t.w;
    } else if constexpr (BITS == 8) {
        const uint32_t w = static_cast<const uint32_t*>(in)[p];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t b = (w >> (8 * e)) & 0xFFu;
            q[e] = SIGNED ? static_cast<int32_t>(static_cast<int8_t>(b)) : static_cast<int32_t>(b);
        }
    } else {
        uint32_t w;  // the 4 * BITS bits of the piece, at bit 0
        if constexpr (BITS == 4) w = static_cast<const uint16_t*>(in)[p];
        if constexpr (BITS == 2) w = static_cast<const uint8_t*>(in)[p];
        if constexpr (BITS == 1) w = static_cast<const uint8_t*>(in)[p >> 1] >> (4 * (p & 1));
#pragma unroll
        for (int e = 0; e < 4; ++e) q[e] = static_cast<int32_t>((w >> (e * BITS)) & ((1u << BITS) - 1u));
    }
}

template <int BITS, bool SIGNED>
__global__ __launch_bounds__(256) void dequantize_pieces_kernel(const void* __restrict__ in, float* __restrict__ out, int64_t pieces,
                                                                Pieces ps, Params pr) {
    constexpr int kFlight = 4;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const bool has_zero = pr.zeros != nullptr;
    for (int64_t p0 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; p0 < pieces; p0 += kFlight * stride) {
        int32_t q[kFlight][4];
        float scale[kFlight], zero[kFlight];
#pragma unroll
        for (int j = 0; j < kFlight; ++j) {
            const int64_t p = p0 + j * stride;
            if (p < pieces) {
                load_piece<BITS, SIGNED>(in, p, q[j]);
                const int64_t b = piece_block(ps, 4 * p);
                scale[j] = pr.scales[pr.scale_is_scalar ? 0 : b];
                zero[j] = has_zero ? pr.zeros[pr.zero_is_scalar ? 0 : b] : 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < kFlight; ++j) {
            const int64_t p = p0 + j * stride;
            if (p < pieces)
                nt_store(reinterpret_cast<float4*>(out) + p, dequantize_one(q[j][0], scale[j], zero[j]), dequantize_one(q[j][1], scale[j], zero[j]),
                         dequantize_one(q[j][2], scale[j], zero[j]), dequantize_one(q[j][3], scale[j], zero[j]));
        }
    }
}

template <int DT>
__device__ __forceinline__ void load_piece_floats(const void* x, int64_t p, float v[4]) {
    if constexpr (DT == TPQ_DTYPE_F32) {
        const uint4 t = nt_load(static_cast<const uint4*>(x) + p);
        v[0] = __builtin_bit_cast(float, t.x); v[1] = __builtin_bit_cast(float, t.y);
        v[2] = __builtin_bit_cast(float, t.z); v[3] = __builtin_bit_cast(float, t.w);
    } else {
        const uint2 t = nt_load(static_cast<const uint2*>(x) + p);
        v[0] = Elem<DT>::load(static_cast<uint16_t>(t.x)); v[1] = Elem<DT>::load(static_cast<uint16_t>(t.x >> 16));
        v[2] = Elem<DT>::load(static_cast<uint16_t>(t.y)); v[3] = Elem<DT>::load(static_cast<uint16_t>(t.y >> 16));
    }
}

// Every lane of a wavefront must call this together (the 1-bit storage pairs neighbouring lanes);
// `live` says whether piece p exists.
template <int BITS>
__device__ __forceinline__ void store_piece(void* out, int64_t p, bool live, const int32_t q[4]) {
    if constexpr (BITS == 32) {
        if (live) static_cast<int4*>(out)[p] = make_int4(q[0], q[1], q[2], q[3]);
    } else if constexpr (BITS == 8) {
        const uint32_t w = (static_cast<uint32_t>(q[0]) & 0xFFu) | ((static_cast<uint32_t>(q[1]) & 0xFFu) << 8) |
                           ((static_cast<uint32_t>(q[2]) & 0xFFu) << 16) | (static_cast<uint32_t>(q[3]) << 24);
        if (live) static_cast<uint32_t*>(out)[p] = w;
    } else {
        // the clamp keeps every code inside its field, as in the reference nothing is masked
        uint32_t w = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) w |= static_cast<uint32_t>(q[e]) << (e * BITS);
        if constexpr (BITS == 4) { if (live) static_cast<uint16_t*>(out)[p] = static_cast<uint16_t>(w); }
        if constexpr (BITS == 2) { if (live) static_cast<uint8_t*>(out)[p] = static_cast<uint8_t>(w); }
        if constexpr (BITS == 1) {
            // pieces 2i and 2i+1 share a byte and sit in neighbouring lanes (the thread index and the
            // piece index have the same parity): the even lane stores both nibbles
            const uint32_t mine = live ? w : 0u;
            const uint32_t other = __shfl_xor(mine, 1, kWave);
            if (live && (p & 1) == 0) static_cast<uint8_t*>(out)[p >> 1] = static_cast<uint8_t>(mine | (other << 4));
        }
    }
}

template <int DT, int BITS>
__global__ __launch_bounds__(256) void quantize_pieces_kernel(const void* __restrict__ x, void* __restrict__ out, int64_t pieces,
                                                              Pieces ps, Params pr) {
    constexpr int kFlight = 4;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;  // even: a piece keeps the parity of its thread
    const bool has_zero = pr.zeros != nullptr;
    // whole wavefronts stay in the loop together: the bound is rounded up to the wavefront
    const int64_t first = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    for (int64_t p0 = first; (p0 & ~int64_t{kWave - 1}) < pieces; p0 += kFlight * stride) {
        float v[kFlight][4], inv[kFlight], zero[kFlight];
#pragma unroll
        for (int j = 0; j < kFlight; ++j) {
            const int64_t p = p0 + j * stride;
            if (p < pieces) {
                load_piece_floats<DT>(x, p, v[j]);
                const int64_t b = piece_block(ps, 4 * p);
                inv[j] = pr.scales[pr.scale_is_scalar ? 0 : b];
                zero[j] = has_zero ? pr.zeros[pr.zero_is_scalar ? 0 : b] : 0.0f;
            } else {
                v[j][0] = v[j][1] = v[j][2] = v[j][3] = 0.0f;
                inv[j] = 1.0f;
                zero[j] = 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < kFlight; ++j) {
            const int64_t p = p0 + j * stride;
            const float r = inverse_of(inv[j]);
            int32_t q[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) q[e] = quantize_one<(BITS < 8)>(v[j][e], r, zero[j], has_zero, pr.qmin, pr.qmax);
            store_piece<BITS>(out, p, p < pieces, q);
        }
    }
}

// General grid: one thread per output byte (one element, or `pack` elements of a packed storage).
template <int DT, int BITS>
__global__ __launch_bounds__(256) void quantize_grid_kernel(const void* __restrict__ x, void* __restrict__ out, int64_t numel,
                                                            Grid grid, Params pr) {
    using S = typename Elem<DT>::storage;
    constexpr int pack = BITS < 8 ? 8 / BITS : 1;
    const int64_t units = (numel + pack - 1) / pack;
    const bool has_zero = pr.zeros != nullptr;
    for (int64_t u = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; u < units;
         u += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        uint32_t value = 0;
        for (int lane = 0; lane < pack && u * pack + lane < numel; ++lane) {
            const int64_t i = u * pack + lane;
            const int64_t b = block_of(grid, i);
            const float inv = inverse_of(pr.scales[pr.scale_is_scalar ? 0 : b]);
            const float zero = has_zero ? pr.zeros[pr.zero_is_scalar ? 0 : b] : 0.0f;
            const int32_t q = quantize_one<(BITS < 8)>(Elem<DT>::load(static_cast<const S*>(x)[i]), inv, zero, has_zero, pr.qmin, pr.qmax);
            if constexpr (BITS == 32) static_cast<int32_t*>(out)[i] = q;
            else value |= ((static_cast<uint32_t>(q) & 0xFFu) << (lane * BITS)) & 0xFFu;
        }
        if constexpr (BITS != 32) static_cast<uint8_t*>(out)[u] = static_cast<uint8_t>(value);
    }
}

template <int BITS, bool SIGNED>
__global__ __launch_bounds__(256) void dequantize_grid_kernel(const void* __restrict__ in, float* __restrict__ out, int64_t numel,
                                                              Grid grid, Params pr) {
    constexpr int pack = BITS < 8 ? 8 / BITS : 1;
    constexpr uint32_t mask = BITS < 8 ? (1u << BITS) - 1u : 0xFFu;
    const bool has_zero = pr.zeros != nullptr;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        int32_t code;
        if constexpr (BITS == 32) {
            code = static_cast<const int32_t*>(in)[i];
        } else {
            const uint32_t field = (static_cast<const uint8_t*>(in)[i / pack] >> ((i % pack) * BITS)) & mask;
            code = SIGNED ? static_cast<int32_t>(static_cast<int8_t>(field)) : static_cast<int32_t>(field);
        }
        const int64_t b = block_of(grid, i);
        out[i] = dequantize_one(code, pr.scales[pr.scale_is_scalar ? 0 : b], has_zero ? pr.zeros[pr.zero_is_scalar ? 0 : b] : 0.0f);
    }
}

unsigned grid_for(int64_t work_items) {
    const int64_t blocks = (work_items + 255) / 256;
    return static_cast<unsigned>(blocks < 1 ? 1 : blocks > (1 << 20) ? (1 << 20) : blocks);
}

int check_params(const char* op, const Plan& plan, int64_t n_scales, int64_t n_zeros) {
    TPQ_REQUIRE(n_scales == plan.num_blocks || n_scales == 1, TPQ_ERR_INVALID_VALUE,
                "%s: scales must have one entry per block (%lld blocks, got %lld)", op, static_cast<long long>(plan.num_blocks),
                static_cast<long long>(n_scales));
    TPQ_REQUIRE(n_zeros == 0 || n_zeros == plan.num_blocks || n_zeros == 1, TPQ_ERR_INVALID_VALUE,
                "%s: zero_points must have one entry per block, or be a scalar", op);
    return TPQ_OK;
}

int log2_if_power_of_two(int64_t v) {
    if (v <= 0 || (v & (v - 1)) != 0) return -1;
    int s = 0;
    while ((int64_t{1} << s) < v) ++s;
    return s;
}

Pieces pieces_of(const Plan& plan, const Params& pr) {
    const Runs& r = plan.runs;
    return {r.K, r.g, r.G, log2_if_power_of_two(r.K), log2_if_power_of_two(r.g), plan.numel < (int64_t{1} << 31),
            !(pr.scale_is_scalar && (pr.zeros == nullptr || pr.zero_is_scalar)) && plan.num_blocks > 1};
}

template <int DT>
int launch_quantize(int bits, bool runs_ok, const void* x, void* out, const Plan& plan, const Params& pr, hipStream_t s) {
    const int64_t n = plan.numel;
    const Pieces ps = pieces_of(plan, pr);
    const bool pieces_ok = runs_ok && plan.runs.K % 4 == 0 && plan.runs.g % 4 == 0;
#define TPQ_AQ_CASE(BITS)                                                                                         \
    case BITS:                                                                                                    \
        if (pieces_ok) quantize_pieces_kernel<DT, BITS><<<grid_for((n / 4 + 3) / 4), 256, 0, s>>>(x, out, n / 4, ps, pr); \
        else if (runs_ok) quantize_runs_kernel<DT, BITS><<<grid_for((n + kChunk - 1) / kChunk), 256, 0, s>>>(x, out, n, plan.runs, pr); \
        else quantize_grid_kernel<DT, BITS><<<grid_for(n), 256, 0, s>>>(x, out, n, plan.grid, pr);                \
        break;
    switch (bits) {
        TPQ_AQ_CASE(8)
        TPQ_AQ_CASE(32)
        TPQ_AQ_CASE(4)
        TPQ_AQ_CASE(2)
        TPQ_AQ_CASE(1)
    }
#undef TPQ_AQ_CASE
    return check_launch("tpq_quantize_affine");
}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int tpq_quantize_affine(const void* x, int x_dtype, int ndim, const int64_t* sizes, const int64_t* block_size,
                                   const float* scales, int64_t n_scales, const float* zero_points, int64_t n_zeros,
                                   int storage, int64_t quant_min, int64_t quant_max, void* out, void* stream) {
    Storage st;
    TPQ_REQUIRE(storage_of(storage, &st), TPQ_ERR_INVALID_TYPE, "quantize_affine(): expected a quantized dtype, got storage tag %d", storage);
    TPQ_REQUIRE(x_dtype == TPQ_DTYPE_F32 || x_dtype == TPQ_DTYPE_F16 || x_dtype == TPQ_DTYPE_BF16, TPQ_ERR_INVALID_TYPE,
                "quantize_affine(): unsupported input dtype tag %d", x_dtype);
    TPQ_REQUIRE(ndim == 0 || (sizes != nullptr && block_size != nullptr), TPQ_ERR_INVALID_VALUE, "quantize_affine(): null shape");
    Plan plan;
    if (int rc = make_plan("quantize_affine()", ndim, sizes, block_size, &plan)) return rc;
    if (int rc = check_params("quantize_affine()", plan, n_scales, n_zeros)) return rc;
    const int64_t qmin = quant_min < quant_max ? quant_min : st.lo;
    const int64_t qmax = quant_max > quant_min ? quant_max : st.hi;
    TPQ_REQUIRE(qmin >= st.lo && qmax <= st.hi, TPQ_ERR_INVALID_VALUE, "quantize(): quantization range does not fit the output storage");
    if (plan.numel == 0) return TPQ_OK;
    TPQ_REQUIRE(x != nullptr && out != nullptr && scales != nullptr && (n_zeros == 0 || zero_points != nullptr), TPQ_ERR_INVALID_VALUE,
                "quantize_affine(): null pointer");
    const Params pr = {scales, n_zeros ? zero_points : nullptr, n_scales == 1, n_zeros == 1, static_cast<int32_t>(qmin), static_cast<int32_t>(qmax)};
    const bool runs_ok = plan.as_runs && aligned(x, 16) && aligned(out, 16);
    auto s = static_cast<hipStream_t>(stream);
    switch (x_dtype) {
        case TPQ_DTYPE_F32: return launch_quantize<TPQ_DTYPE_F32>(st.bits, runs_ok, x, out, plan, pr, s);
        case TPQ_DTYPE_F16: return launch_quantize<TPQ_DTYPE_F16>(st.bits, runs_ok, x, out, plan, pr, s);
        default: return launch_quantize<TPQ_DTYPE_BF16>(st.bits, runs_ok, x, out, plan, pr, s);
    }
}

TPQ_EXPORT int tpq_dequantize_affine(const void* codes, int storage, int ndim, const int64_t* sizes, const int64_t* block_size,
                                     const float* scales, int64_t n_scales, const float* zero_points, int64_t n_zeros,
                                     float* out, void* stream) {
    Storage st;
    TPQ_REQUIRE(storage_of(storage, &st), TPQ_ERR_INVALID_TYPE, "dequantize_affine(): expected a quantized tensor, got storage tag %d", storage);
    TPQ_REQUIRE(ndim == 0 || (sizes != nullptr && block_size != nullptr), TPQ_ERR_INVALID_VALUE, "dequantize_affine(): null shape");
    Plan plan;
    if (int rc = make_plan("dequantize_affine()", ndim, sizes, block_size, &plan)) return rc;
    if (int rc = check_params("dequantize_affine()", plan, n_scales, n_zeros)) return rc;
    if (plan.numel == 0) return TPQ_OK;
    TPQ_REQUIRE(codes != nullptr && out != nullptr && scales != nullptr && (n_zeros == 0 || zero_points != nullptr), TPQ_ERR_INVALID_VALUE,
                "dequantize_affine(): null pointer");
    const Params pr = {scales, n_zeros ? zero_points : nullptr, n_scales == 1, n_zeros == 1, 0, 0};
    const bool runs_ok = plan.as_runs && aligned(codes, 16) && aligned(out, 16);
    auto s = static_cast<hipStream_t>(stream);
    const int64_t n = plan.numel;
    const Pieces ps = pieces_of(plan, pr);
    const bool pieces_ok = runs_ok && plan.runs.K % 4 == 0 && plan.runs.g % 4 == 0;
#define TPQ_ADQ_CASE(TAG, BITS, SIGNED)                                                                                         \
    case TAG:                                                                                                                   \
        if (pieces_ok) dequantize_pieces_kernel<BITS, SIGNED><<<grid_for((n / 4 + 3) / 4), 256, 0, s>>>(codes, out, n / 4, ps, pr); \
        else if (runs_ok) dequantize_runs_kernel<BITS, SIGNED><<<grid_for((n + kChunk - 1) / kChunk), 256, 0, s>>>(codes, out, n, plan.runs, pr); \
        else dequantize_grid_kernel<BITS, SIGNED><<<grid_for(n), 256, 0, s>>>(codes, out, n, plan.grid, pr);                    \
        break;
    switch (storage) {
        TPQ_ADQ_CASE(TPQ_STORAGE_I8, 8, true)
        TPQ_ADQ_CASE(TPQ_STORAGE_U8, 8, false)
        TPQ_ADQ_CASE(TPQ_STORAGE_I32, 32, true)
        TPQ_ADQ_CASE(TPQ_STORAGE_U4X2, 4, false)
        TPQ_ADQ_CASE(TPQ_STORAGE_U2X4, 2, false)
        TPQ_ADQ_CASE(TPQ_STORAGE_U1X8, 1, false)
    }
#undef TPQ_ADQ_CASE
    return check_launch("tpq_dequantize_affine");
}
