// Measurement probe: a pure read of a device buffer, the ceiling that the bandwidth-bound decode kernels are held
// against.  It does no arithmetic on what it reads beyond an exclusive-or that keeps the loads alive.
//
// Pattern: every wavefront load is 1 KB contiguous (16 bytes per lane); a wavefront issues all its loads of a round
// before it looks at the first one, so the whole buffer is requested within the first microsecond when
// workgroups x wavefronts x loads x 1 KB covers it.  Blocks of 1 KB are dealt to the wavefronts either interleaved
// (wavefront w takes blocks w, w + W, w + 2 W, ...: neighbouring wavefronts read neighbouring kilobytes) or as one
// contiguous run per wavefront.
//
// Built into a library of its own (libtpq_probe.so, loaded by the benchmark only): it is a measuring instrument, not an
// operator, and the kernel library's interface lists operators only.  Signature:
//   int tpq_probe_read(const void* src, int64_t bytes, int workgroups, int waves, int loads_in_flight, int contiguous,
//                      void* sink, void* stream)
// reads `bytes` (a multiple of 1024) of device memory with `workgroups` x `waves` wavefronts that each keep
// `loads_in_flight` (2, 4, 8, 12, 16 or 24) 1 KB loads outstanding; `contiguous` = 1 gives every wavefront one contiguous
// run, 0 interleaves the wavefronts kilobyte by kilobyte; `contiguous` in 2..1024 selects the access pattern of the
// column-per-lane decode kernel for a packed int4 weight with K = 128 x contiguous (one workgroup per 64 columns,
// `workgroups` ignored, 16-byte loads that touch eight 128-byte lines per wavefront; bytes must then be a multiple of
// 512 x contiguous).  bytes = 0 launches an empty kernel of the same grid.  `sink`: 256 bytes that are practically never written.
#include <cstdarg>
#include <cstdio>

#include "tpq_common.h"

namespace tpq {
// the error plumbing of tpq_common.h, for this library alone
char* error_buffer() {
    static thread_local char buffer[512] = "";
    return buffer;
}
int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}
namespace {

template <int LOADS>
__global__ __launch_bounds__(1024) void read_probe_kernel(const uint4* __restrict__ src, int64_t blocks, int contiguous,
                                                          uint32_t* __restrict__ sink) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t waves_per_group = blockDim.x / kWave;
    const int64_t wave = blockIdx.x * waves_per_group + (threadIdx.x >> 6);
    const int64_t total_waves = gridDim.x * waves_per_group;
    const int64_t per_wave = (blocks + total_waves - 1) / total_waves;
    uint32_t acc = 0;
    for (int64_t r = 0; r < per_wave; r += LOADS) {
        uint4 v[LOADS];
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            int64_t b = contiguous ? wave * per_wave + r + i : (r + i) * total_waves + wave;
            const bool live = r + i < per_wave && b < blocks;
            b = live ? b : 0;  // past the end: a valid block, not counted
            v[i] = nt_load(src + b * kWave + lane);
            if (!live) v[i] = make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < LOADS; ++i) acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    }
    if (acc == 0x9E3779B9u && sink != nullptr) sink[wave & 63] = acc;  // practically never: keeps the loads alive
}

// The access pattern of the column-per-lane decode kernel, without its arithmetic: workgroup = 64 columns = eight
// tiles of the packed layout (k_super x 128 bytes each), 16 wavefronts, wavefront w reads the chunks (four k-tiles)
// w, w + 16, ...; lane l = row l % 8 of tile l / 8, 16 bytes per k-tile: a wavefront load touches eight 128-byte
// lines that lie k_super x 128 bytes apart.  All loads of a wavefront are issued before the first use.
template <int CHUNKS>
__global__ __launch_bounds__(1024) void read_probe_columns_kernel(const uint4* __restrict__ src, int n_tiles, int k_super,
                                                                  uint32_t* __restrict__ sink) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    int tile = blockIdx.x * 8 + (lane >> 3);
    tile = tile < n_tiles ? tile : n_tiles - 1;
    const uint4* base = src + (static_cast<size_t>(tile) * k_super) * 8 + (lane & 7);
    const int n_chunks = k_super / 4;
    uint32_t acc = 0;
    for (int c0 = wave; c0 < n_chunks; c0 += waves * CHUNKS) {
        uint4 v[CHUNKS][4];
#pragma unroll
        for (int u = 0; u < CHUNKS; ++u) {
            int c = c0 + u * waves;
            c = c < n_chunks ? c : n_chunks - 1;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[u][i] = nt_load(base + static_cast<size_t>(c * 4 + i) * 8);
        }
#pragma unroll
        for (int u = 0; u < CHUNKS; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc ^= v[u][i].x ^ v[u][i].y ^ v[u][i].z ^ v[u][i].w;
    }
    if (acc == 0x9E3779B9u && sink != nullptr) sink[wave & 63] = acc;
}

__global__ void empty_probe_kernel() {}

}  // namespace
}  // namespace tpq

using namespace tpq;

TPQ_EXPORT int tpq_probe_read(const void* src, int64_t bytes, int workgroups, int waves, int loads_in_flight, int contiguous,
                              void* sink, void* stream) {
    TPQ_REQUIRE(bytes >= 0 && bytes % 1024 == 0, TPQ_ERR_INVALID_VALUE, "probe_read: bytes must be a multiple of 1024");
    TPQ_REQUIRE(workgroups >= 1 && waves >= 1 && waves <= 16, TPQ_ERR_INVALID_VALUE, "probe_read: 1..16 wavefronts per workgroup");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (bytes == 0) {  // the cost of a launch alone
        empty_probe_kernel<<<workgroups, waves * kWave, 0, s>>>();
        return check_launch("probe_read (empty)");
    }
    TPQ_REQUIRE(src && aligned(src, 16), TPQ_ERR_INVALID_VALUE, "probe_read: source must be 16-byte aligned");
    if (contiguous >= 2) {  // the column-per-lane pattern: `workgroups` is ignored, one per 64 columns; K = 128 x contiguous
        TPQ_REQUIRE(contiguous <= 1024, TPQ_ERR_INVALID_VALUE, "probe_read: column pattern: contiguous = K / 128 must be at most 1024");
        TPQ_REQUIRE(loads_in_flight == 2 || loads_in_flight == 4 || loads_in_flight == 8 || loads_in_flight == 12 || loads_in_flight == 16 || loads_in_flight == 24,
                    TPQ_ERR_INVALID_VALUE, "probe_read: loads in flight must be 2, 4, 8, 12, 16 or 24");
        const int k_super = contiguous * 4;  // contiguous = K / 128
        TPQ_REQUIRE(bytes % (static_cast<int64_t>(k_super) * 128) == 0 && bytes / (static_cast<int64_t>(k_super) * 128) <= 0x7FFFFFF,
                    TPQ_ERR_INVALID_VALUE, "probe_read: column pattern: bytes must be whole tile rows of 512 x contiguous bytes");
        const int n_tiles = static_cast<int>(bytes / (static_cast<int64_t>(k_super) * 128));
        const dim3 g((n_tiles + 7) / 8), b(static_cast<unsigned>(waves * kWave));
        if (loads_in_flight >= 8) read_probe_columns_kernel<2><<<g, b, 0, s>>>(static_cast<const uint4*>(src), n_tiles, k_super, static_cast<uint32_t*>(sink));
        else read_probe_columns_kernel<1><<<g, b, 0, s>>>(static_cast<const uint4*>(src), n_tiles, k_super, static_cast<uint32_t*>(sink));
        return check_launch("probe_read (columns)");
    }
    const int64_t blocks = bytes / 1024;
    const uint4* p = static_cast<const uint4*>(src);
    uint32_t* out = static_cast<uint32_t*>(sink);
    const dim3 grid(static_cast<unsigned>(workgroups)), block(static_cast<unsigned>(waves * kWave));
    switch (loads_in_flight) {
        case 2: read_probe_kernel<2><<<grid, block, 0, s>>>(p, blocks, contiguous, out); break;
        case 4: read_probe_kernel<4><<<grid, block, 0, s>>>(p, blocks, contiguous, out); break;
        case 8: read_probe_kernel<8><<<grid, block, 0, s>>>(p, blocks, contiguous, out); break;
        case 12: read_probe_kernel<12><<<grid, block, 0, s>>>(p, blocks, contiguous, out); break;
        case 16: read_probe_kernel<16><<<grid, block, 0, s>>>(p, blocks, contiguous, out); break;
        case 24: read_probe_kernel<24><<<grid, block, 0, s>>>(p, blocks, contiguous, out); break;
        default: return fail(TPQ_ERR_INVALID_VALUE, "probe_read: loads in flight must be 2, 4, 8, 12, 16 or 24");
    }
    return check_launch("probe_read");
}
