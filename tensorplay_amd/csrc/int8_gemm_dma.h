// int8 GEMM for large problems: 256 x 128 tile per workgroup, multi-stage LDS
// ring filled by direct global -> LDS loads, fragment reads one k-substep
// ahead of the matrix cores, and an epilogue that goes back through LDS so
// that the result leaves in 16-byte row-contiguous stores.
//
// Main loop.  k-step 64 bytes, 4 wavefronts of 128 (m) x 64 (n) = 4 x 2 blocks
// of v_mfma_i32_32x32x32_i8.  LDS layout of a stage: row r holds its four
// 16-byte chunks at position chunk ^ swz(r) (conflict-free for the fragment
// reads).  A direct load (global_load_lds_dwordx4) writes lane l's 16 bytes to
// slot l of a 1 KB LDS region whose base is wave-uniform, so the swizzle is
// applied on the global side: lane l fetches the chunk that belongs in slot l.
// A stage is 24 wave-level loads, six per wavefront, and STAGES-1 stages are
// in flight while one is being multiplied.
//
// Measured on MI355X: LDS serves about 98 bytes/clock/CU to four wavefronts
// issuing ds_read_b128, and this tiling reads 96 bytes per clock of MFMA work,
// so the fragment reads have to overlap the MFMAs completely: the reads of
// substep s+1 are issued before the MFMAs of substep s.
//
// Ordering.  Vector loads of a wavefront complete in order: once at most
// (STAGES-2)*6 are outstanding, this wavefront's share of the oldest stage has
// landed.  The workgroup barrier that follows makes every wavefront's share
// visible and proves that everybody is done with the buffer the next direct
// load overwrites.  The barrier is the bare instruction: __syncthreads() would
// also drain all outstanding direct loads, i.e. the prefetched stages.
//
// Epilogue.  The MFMA is issued with the W fragment as its first operand, so a
// lane ends up with 4 consecutive n for one m in each accumulator quad; those
// are scaled, converted and written to an LDS image of the output tile, which
// the workgroup then stores row by row, 16 bytes per lane.
//
// Requires K % 64 == 0 and 16-byte aligned operands.  Edges in M and N are
// handled by clamping source rows and masking the stores.
#pragma once

#include <cstdlib>

#include "int8_gemm_kernel.h"

namespace tpq {
namespace {

typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* global_void_ptr;

constexpr int vmcnt_imm(int n) {  // s_waitcnt immediate: vmcnt = n, expcnt and lgkmcnt untouched
    return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8);
}

// What the tile epilogue writes: raw sums, or (float(acc) * rs[m]) * cs[n] (+ bias[n]) in OutT.
struct TileInt32 {
    using out_t = int32_t;
    static constexpr bool kScaled = false;
    int32_t* out;
    const float* rs;
    const float* cs;
    const float* bias;
    static __device__ __forceinline__ int32_t convert(int acc, float, float, float, bool) { return acc; }
};

template <int DT>
struct TileDequant {
    using out_t = typename Elem<DT>::storage;
    static constexpr bool kScaled = true;
    out_t* out;
    const float* rs;
    const float* cs;
    const float* bias;
    static __device__ __forceinline__ out_t convert(int acc, float r, float c, float b, bool has_bias) {
        float f = __fmul_rn(__fmul_rn(static_cast<float>(acc), r), c);
        if (has_bias) f = __fadd_rn(f, b);
        return Elem<DT>::store(f);
    }
};

template <int STAGES, int KSPLIT, class Tile>
__global__ __launch_bounds__(256 * KSPLIT) void int8_gemm_dma_kernel(const int8_t* __restrict__ A,
                                                            const int8_t* __restrict__ W, int M, int N,
                                                            int K, Tile tile, int vector_stores) {
    using out_t = typename Tile::out_t;
    constexpr int BM = 256, BN = 128, WM = 128, WN = 64, TM = 4, TN = 2;
    constexpr int kStageChunks = (BM + BN) * kChunksPerRow;  // 1536 x 16 B = 24 KB
    constexpr int kThreads = 256 * KSPLIT, kWaves = 4 * KSPLIT;
    constexpr int kLoadsPerWave = kStageChunks / kWave / kWaves;  // wave-level loads per stage: 6 or 3
    constexpr int kUnitsPerStage = 2 / KSPLIT;               // 32-byte k-substeps a wavefront multiplies per stage
    constexpr int kPerChunk = 16 / sizeof(out_t);            // outputs per 16 bytes
    constexpr int kPitch = BN * sizeof(out_t) + 16;          // bytes per row of the output image
    constexpr int kRingBytes = STAGES * kStageChunks * 16;
    constexpr int kImageBytes = BM * kPitch;
    constexpr int kPartialBytes = KSPLIT > 1 ? 4 * 128 * kWave * 4 : 0;  // accumulators of the second k-half
    constexpr int kScaleOffset = (kRingBytes > kImageBytes ? kRingBytes : kImageBytes) > kPartialBytes
                                     ? (kRingBytes > kImageBytes ? kRingBytes : kImageBytes) : kPartialBytes;
    extern __shared__ uint4 ring[];                          // [STAGES][kStageChunks], later the image
    char* lds_bytes = reinterpret_cast<char*>(ring);
    float* cs_lds = reinterpret_cast<float*>(lds_bytes + kScaleOffset);  // [BN] column scales, [BN] bias

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kh = wave >> 2;               // which k-substep of every stage this wavefront multiplies (KSPLIT = 2)
    const int wm = (wave >> 1) & 1, wn = wave & 1;

    // Workgroups are dealt to the 8 XCDs round-robin (workgroup id mod 8), each with its own L2:
    // give every XCD a compact patch of tiles, as close to square in bytes as the grid allows,
    // so that the A and W panels it streams are shared by as many of its workgroups as possible.
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tile_m, tile_n;
    {
        const int id = blockIdx.x, total = tiles_m * tiles_n;
        if (total % 8 == 0 && tiles_m % 2 == 0 && tiles_n % 4 == 0) {
            const int xcd = id & 7, local = id >> 3;         // local: index inside the XCD's patch
            const int pm = tiles_m / 2, pn = tiles_n / 4;    // patch: (tiles_m/2) x (tiles_n/4)
            tile_m = (xcd & 1) * pm + local % pm;
            tile_n = (xcd >> 1) * pn + local / pm;
        } else {
            tile_m = id % tiles_m;
            tile_n = id / tiles_m;
        }
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int nk = K / kBK;

    if (Tile::kScaled && tid < BN) {  // column scales and bias of this tile: read once, used in the epilogue
        const int n = n0 + tid < N ? n0 + tid : N - 1;
        cs_lds[tid] = tile.cs[n];
        cs_lds[BN + tid] = tile.bias ? tile.bias[n] : 0.0f;
    }

    // what lane l of wave-level load i fetches: slot (wave*6 + i)*64 + l of the stage
    const int8_t* src[kLoadsPerWave];
#pragma unroll
    for (int i = 0; i < kLoadsPerWave; ++i) {
        const int row = (wave * kLoadsPerWave + i) * 16 + (lane >> 2);   // stage row 0..383
        const int chunk = (lane & 3) ^ swz(row);
        if (row < BM) {
            int gr = m0 + row;
            gr = gr < M ? gr : M - 1;
            src[i] = A + static_cast<size_t>(gr) * K + chunk * 16;
        } else {
            int gr = n0 + row - BM;
            gr = gr < N ? gr : N - 1;
            src[i] = W + static_cast<size_t>(gr) * K + chunk * 16;
        }
    }
    auto issue = [&](int kt) {
        uint4* stage = ring + (kt % STAGES) * kStageChunks;
#pragma unroll
        for (int i = 0; i < kLoadsPerWave; ++i)
            __builtin_amdgcn_global_load_lds((global_void_ptr)(src[i] + static_cast<size_t>(kt) * kBK),
                                             (lds_void_ptr)(stage + (wave * kLoadsPerWave + i) * kWave), 16, 0, 0);
    };
    // this wavefront's loads of stage kt are complete: at the points where it is called the
    // stages up to kt + YOUNGER have been issued, so that many may still be outstanding
    auto landed = [&](int kt, auto younger) {
        constexpr int kYounger = decltype(younger)::value;
        if (nk - 1 - kt >= kYounger) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kYounger * kLoadsPerWave));
        else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    const int frag_row = lane & 31, frag_half = lane >> 5;
    int a_off[TM], b_off[TN], a_swz[TM], b_swz[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int r = wm * WM + i * 32 + frag_row;
        a_off[i] = r * kChunksPerRow;
        a_swz[i] = swz(r);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int r = BM + wn * WN + j * 32 + frag_row;
        b_off[j] = r * kChunksPerRow;
        b_swz[j] = swz(r);
    }
    auto read_frags = [&](int kt, int ks, v4i (&fa)[TM], v4i (&fb)[TN]) {
        const uint4* stage = ring + (kt % STAGES) * kStageChunks;
        const int chunk = ks * 2 + frag_half;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = __builtin_bit_cast(v4i, stage[a_off[i] + (chunk ^ a_swz[i])]);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j] = __builtin_bit_cast(v4i, stage[b_off[j] + (chunk ^ b_swz[j])]);
    };
    auto multiply = [&](const v4i (&fa)[TM], const v4i (&fb)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)  // W fragment first: accumulator rows run along n
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0);
    };

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < nk) issue(s);

    // Buffers in use while stage kt is multiplied: kt (being read), kt+1 .. kt+STAGES-2 (landed
    // or in flight).  The barrier sits in the middle of a stage; when a wavefront passes it,
    // all wavefronts have consumed their reads of stage kt-1, whose buffer takes stage
    // kt+STAGES-1.
    v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    landed(0, std::integral_constant<int, STAGES - 2>{});
    asm volatile("s_barrier" ::: "memory");
    // moving on to stage kt: wait for it, meet, refill the buffer stage kt-2 was read from
    auto advance = [&](int kt) {
        landed(kt, std::integral_constant<int, STAGES - 3>{});
        asm volatile("s_barrier" ::: "memory");
        if (kt + STAGES - 2 < nk) issue(kt + STAGES - 2);
    };
    if constexpr (KSPLIT == 1) {
        read_frags(0, 0, fa0, fb0);
        for (int kt = 0; kt < nk; ++kt) {
            read_frags(kt, 1, fa1, fb1);  // second half of this stage, in flight during the first MFMAs
            multiply(fa0, fb0);
            if (kt + 1 < nk) {
                advance(kt + 1);
                read_frags(kt + 1, 0, fa0, fb0);  // first half of the next stage, in flight during the second MFMAs
            }
            multiply(fa1, fb1);
        }
    } else {  // one substep (kh) per stage and wavefront; fragments of the next stage in flight during the MFMAs
        read_frags(0, kh, fa0, fb0);
        for (int kt = 0; kt < nk; kt += 2) {
            if (kt + 1 < nk) {
                advance(kt + 1);
                read_frags(kt + 1, kh, fa1, fb1);
            }
            multiply(fa0, fb0);
            if (kt + 1 < nk) {
                if (kt + 2 < nk) {
                    advance(kt + 2);
                    read_frags(kt + 2, kh, fa0, fb0);
                }
                multiply(fa1, fb1);
            }
        }
    }

    // ---- epilogue: scale, convert, image in LDS, row-contiguous stores -----------------------------
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // ring no longer needed
    if constexpr (KSPLIT > 1) {  // fold the second k-half into the first through LDS
        int4* part = reinterpret_cast<int4*>(lds_bytes) + (wave & 3) * (TM * TN * 4) * kWave + lane;
        if (kh == 1) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        part[((i * TN + j) * 4 + q) * kWave] = make_int4(acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
        }
        __syncthreads();
        if (kh == 0) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int4 o = part[((i * TN + j) * 4 + q) * kWave];
                        acc[i][j][4 * q] += o.x; acc[i][j][4 * q + 1] += o.y; acc[i][j][4 * q + 2] += o.z; acc[i][j][4 * q + 3] += o.w;
                    }
        }
        __syncthreads();  // partials consumed before the image overwrites them
    }
    if (kh == 0) {
    float rs_r[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * WM + i * 32 + frag_row;
        rs_r[i] = Tile::kScaled ? tile.rs[m < M ? m : M - 1] : 0.0f;
    }
    const bool has_bias = tile.bias != nullptr;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int n_local = wn * WN + j * 32 + 8 * q + 4 * frag_half;  // 4 consecutive columns
            float c4[4] = {0, 0, 0, 0}, b4[4] = {0, 0, 0, 0};
            if (Tile::kScaled) {
                const float4 c = *reinterpret_cast<const float4*>(cs_lds + n_local);
                const float4 b = *reinterpret_cast<const float4*>(cs_lds + BN + n_local);
                c4[0] = c.x; c4[1] = c.y; c4[2] = c.z; c4[3] = c.w;
                b4[0] = b.x; b4[1] = b.y; b4[2] = b.z; b4[3] = b.w;
            }
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m_local = wm * WM + i * 32 + frag_row;
                out_t vals[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) vals[t] = Tile::convert(acc[i][j][4 * q + t], rs_r[i], c4[t], b4[t], has_bias);
                char* dst = lds_bytes + m_local * kPitch + n_local * sizeof(out_t);
                if constexpr (sizeof(out_t) == 2) {
                    *reinterpret_cast<uint2*>(dst) = make_uint2(vals[0] | (static_cast<uint32_t>(vals[1]) << 16),
                                                                vals[2] | (static_cast<uint32_t>(vals[3]) << 16));
                } else {
                    *reinterpret_cast<uint4*>(dst) = make_uint4(__builtin_bit_cast(uint32_t, vals[0]), __builtin_bit_cast(uint32_t, vals[1]),
                                                                __builtin_bit_cast(uint32_t, vals[2]), __builtin_bit_cast(uint32_t, vals[3]));
                }
            }
        }
    }  // kh == 0
    __syncthreads();
    constexpr int kChunksPerOutRow = BN / kPerChunk;  // 16-byte chunks per image row
    for (int c = tid; c < BM * kChunksPerOutRow; c += kThreads) {
        const int row = c / kChunksPerOutRow, col = (c % kChunksPerOutRow) * kPerChunk;
        const int m = m0 + row, n = n0 + col;
        if (m >= M || n >= N) continue;
        const char* srcp = lds_bytes + row * kPitch + col * sizeof(out_t);
        out_t* dstp = tile.out + static_cast<size_t>(m) * N + n;
        if (vector_stores && n + kPerChunk <= N) {
            *reinterpret_cast<uint4*>(dstp) = *reinterpret_cast<const uint4*>(srcp);
        } else {
            for (int e = 0; e < kPerChunk && n + e < N; ++e) dstp[e] = reinterpret_cast<const out_t*>(srcp)[e];
        }
    }
}

template <int STAGES, int KSPLIT, class Tile>
constexpr size_t dma_lds_bytes() {
    constexpr size_t ring = static_cast<size_t>(STAGES) * (256 + 128) * kBK;
    constexpr size_t image = 256 * (128 * sizeof(typename Tile::out_t) + 16);
    constexpr size_t partial = KSPLIT > 1 ? 4 * 128 * kWave * 4 : 0;
    constexpr size_t body = ring > image ? (ring > partial ? ring : partial) : (image > partial ? image : partial);
    return body + 2 * 128 * sizeof(float);
}

template <int KSPLIT, class Tile>
int launch_dma_split(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Tile tile, hipStream_t s) {
    constexpr int kStages = 5;
    constexpr size_t smem = dma_lds_bytes<kStages, KSPLIT, Tile>();
    const int64_t tiles = ((M + 255) / 256) * ((N + 127) / 128);
    TPQ_REQUIRE(tiles <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "int8 gemm: too many tiles");
    auto kernel = int8_gemm_dma_kernel<kStages, KSPLIT, Tile>;
    static bool configured = false;  // per instantiation: raise the dynamic LDS limit once
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        if (e != hipSuccess) return fail(TPQ_ERR_RUNTIME, "int8 gemm: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
        configured = true;
    }
    const int vector_stores = (N * sizeof(typename Tile::out_t)) % 16 == 0 && aligned(tile.out, 16);
    kernel<<<dim3(static_cast<unsigned>(tiles)), 256 * KSPLIT, smem, s>>>(a, w, static_cast<int>(M), static_cast<int>(N),
                                                                        static_cast<int>(K), tile, vector_stores);
    return check_launch("int8 mfma gemm (dma)");
}

// KSPLIT = 2: eight wavefronts per workgroup, the two k-substeps of every stage go to different
// wavefronts (two per SIMD keep LDS and the matrix cores busier than one).  TPQ_INT8_KSPLIT=1
// selects the four-wavefront variant for comparison runs.
template <class Tile>
int launch_dma(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Tile tile, hipStream_t s) {
    const char* env = std::getenv("TPQ_INT8_KSPLIT");
    if (env && env[0] == '1') return launch_dma_split<1>(a, w, M, N, K, tile, s);
    return launch_dma_split<2>(a, w, M, N, K, tile, s);
}

}  // namespace
}  // namespace tpq
