// int8 GEMM for large problems: 256 x 128 tile per workgroup, three-stage LDS
// ring filled by direct global -> LDS loads of whole 128-byte cache lines,
// fragment reads one k-substep ahead of the matrix cores, and an epilogue
// that goes back through LDS so that the result leaves in 16-byte
// row-contiguous stores.
//
// What bounds it (measured on MI355X, M = 2048, N = K = 4096).  Every
// workgroup pulls (256 + 128) x K bytes through its compute unit's vector
// memory path, 403 MB over the chip.  Filling LDS with nothing else going on
// takes 27.5 us when a row contributes 64 bytes per request and 17.4 us when
// it contributes a whole 128-byte line (8 consecutive lanes of a
// global_load_lds_dwordx4), which is about what the matrix cores need for the
// arithmetic (16 - 20 us depending on clock).  So a stage is 128 bytes of k,
// and the loop is arranged so that fills, fragment reads and MFMAs overlap.
//
// Main loop.  Eight wavefronts: four positions of 128 (m) x 64 (n) = 4 x 2
// blocks of v_mfma_i32_32x32x32_i8, times two k-halves: of the four 32-byte
// k-substeps of a stage a wavefront multiplies two (kh*2, kh*2+1); the two
// partial sums meet in the epilogue.  LDS layout of a stage: row r holds its
// eight 16-byte chunks at position chunk ^ ((r >> 1) & 7), which makes the
// fragment reads conflict-free.  A direct load writes lane l's 16 bytes to slot
// l of a 1 KB region whose base is wave-uniform, so the swizzle is applied on
// the global side: lane l fetches the chunk that belongs in slot l.  A stage is
// 48 wave-level loads, six per wavefront.
//
// Ordering.  Per stage kt a wavefront does
//     request fragments (kt, second substep)
//     multiply (kt, first substep)
//     wait for its own reads of stage kt and for its share of stage kt+1, BARRIER
//     multiply (kt, second substep), and between its MFMAs: request fragments
//     (kt+1, first substep), refill kt's buffer with kt+3
// Passing the barrier proves that every wavefront has finished reading stage kt
// (its buffer may be overwritten) and that every wavefront's share of stage kt+1
// has landed.  Vector loads of a wavefront complete in order, so "my share of
// kt+1 has landed" is "at most the six loads of kt+2 are outstanding".  The
// barrier is the bare instruction: __syncthreads() would also drain all
// outstanding direct loads, i.e. the prefetched stages.  Stages kt+1 .. kt+3
// are in flight or landed while kt is multiplied, 2.5 stage times of lookahead.
//
// Fragment reads and the waits for them are spelled out.  While a direct load
// is in flight the compiler treats the LDS counter as unordered and waits for
// it to reach zero before the first use of ANY fragment, including the reads
// issued a moment ago for the next substep, whose latency the MFMAs are there to
// cover; the steady-state loop is also free of branches for the same reason.
//
// Epilogue.  The two k-halves swap half of their accumulators through LDS, so
// each finishes 64 of the 128 rows of its position.  The MFMA is issued with the
// W fragment as its first operand, so a lane ends up with 4 consecutive n for
// one m in each accumulator quad; those are scaled, converted and written to an
// LDS image of the output tile, which the workgroup then stores row by row, 16
// bytes per lane.
//
// Second form of the main loop (KSPLIT = 0), used below 64 stages per workgroup: eight positions of 64 x 64, every
// wavefront multiplies all four substeps of a stage with the fragments of all four in registers, the barrier in the
// middle of the stage; no exchange of k-halves in the epilogue.
//
// Requires K % 128 == 0 and 16-byte aligned operands.  Edges in M and N are
// handled by clamping source rows and masking the stores.
#pragma once

#include <cstdlib>
#include <type_traits>

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
    static __device__ __forceinline__ float value(int, float, float, float, bool) { return 0.0f; }
    static __device__ __forceinline__ uint32_t pack2(float, float) { return 0; }
};

template <int DT>
struct TileDequant {
    using out_t = typename Elem<DT>::storage;
    static constexpr bool kScaled = true;
    out_t* out;
    const float* rs;
    const float* cs;
    const float* bias;
    static __device__ __forceinline__ float value(int acc, float r, float c, float b, bool has_bias) {
        float f = __fmul_rn(__fmul_rn(static_cast<float>(acc), r), c);
        if (has_bias) f = __fadd_rn(f, b);
        return f;
    }
    static __device__ __forceinline__ out_t convert(int acc, float r, float c, float b, bool has_bias) {
        return Elem<DT>::store(value(acc, r, c, b, has_bias));
    }
    // two results rounded to nearest even and packed, with the hardware's packed conversion
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef float f2_t __attribute__((ext_vector_type(2)));
        const f2_t v = {lo, hi};
        if constexpr (DT == TPQ_DTYPE_BF16) {
            typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
            return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2_t));
        } else {
            typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
            return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, h2_t));
        }
    }
};

// float32 accumulators of a float16 / bfloat16 product, rounded once to the output type (no scales)
template <int DT>
struct TileFloat {
    using out_t = typename Elem<DT>::storage;
    static constexpr bool kScaled = false;
    out_t* out;
    const float* rs;
    const float* cs;
    const float* bias;
    static __device__ __forceinline__ float value(float acc, float, float, float, bool) { return acc; }
    static __device__ __forceinline__ out_t convert(float acc, float, float, float, bool) { return Elem<DT>::store(acc); }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return TileDequant<DT>::pack2(lo, hi); }
};

constexpr int kDmaRowBytes = 128;  // bytes of k per stage: one cache line per row
constexpr int kDmaStages = 3;

#ifdef TPQ_DMA_STAMPS
__device__ unsigned long long g_dma_stamps[8 * 8];
#define TPQ_DMA_STAMP(I) do { if (blockIdx.x == 9 && (threadIdx.x & 63) == 0) g_dma_stamps[(I) * 8 + (threadIdx.x >> 6)] = __builtin_amdgcn_s_memtime(); } while (0)
#else
#define TPQ_DMA_STAMP(I) do { } while (0)
#endif

// KSPLIT = 2: eight wavefronts as described above (four positions x two k-halves).  KSPLIT = 0: eight wavefronts,
// eight positions of 64 x 64, no k split.  KSPLIT = 1: four wavefronts, each multiplying all four substeps of a
// stage (no k-half exchange in the epilogue, one wavefront per SIMD).
template <class Tile, int KSPLIT>
__global__ __launch_bounds__(KSPLIT == 1 ? 256 : 512) void int8_gemm_dma_kernel(const int8_t* __restrict__ A,
                                                            const int8_t* __restrict__ W, int M, int N,
                                                            int K, Tile tile, int vector_stores, int slices) {
    using out_t = typename Tile::out_t;
    constexpr int BM = 256, BN = 128, WM = KSPLIT == 0 ? 64 : 128, WN = 64, TM = WM / 32, TN = 2;
    constexpr int kStageBytes = (BM + BN) * kDmaRowBytes;    // 48 KB
    constexpr int kThreads = KSPLIT == 1 ? 256 : 512, kWaves = kThreads / 64;
    constexpr int kLoads = kStageBytes / 1024 / kWaves;      // wave-level loads per stage and wavefront: 6 or 12
    constexpr int kPerChunk = 16 / sizeof(out_t);            // outputs per 16 bytes
    constexpr int kPitch = BN * sizeof(out_t) + 16;          // bytes per row of the output image
    constexpr int kRingBytes = kDmaStages * kStageBytes;     // 144 KB, covers the image and the exchange area
    static_assert(BM * kPitch <= kRingBytes && 8 * 16 * kWave * 16 <= kRingBytes, "epilogue areas live in the ring");
    extern __shared__ uint4 ring[];                          // [stage][row][128 B], later exchange area and image
    char* lds_bytes = reinterpret_cast<char*>(ring);
    float* cs_lds = reinterpret_cast<float*>(lds_bytes + kRingBytes);  // [BN] column scales, [BN] bias, [BM] row scales
    float* rs_lds = cs_lds + 2 * BN;

    const int tid = threadIdx.x;
    TPQ_DMA_STAMP(0);
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kh = KSPLIT == 2 ? wave >> 2 : 0;  // k-half: substeps 2*kh and 2*kh+1 of every stage
    const int wm = KSPLIT == 0 ? wave >> 1 : (wave >> 1) & 1, wn = wave & 1;

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
    // blockIdx.y = slice of the k range (whole stages, every slice at least one: the launcher sees to it);
    // slice z writes its sums to the z-th [M][N] matrix of the destination
    const int nk_all = K / kDmaRowBytes, nk_slice = (nk_all + slices - 1) / slices;
    const int kt0 = blockIdx.y * nk_slice;
    const int nk = nk_all - kt0 < nk_slice ? nk_all - kt0 : nk_slice;

    // Scales and bias of this tile: asked for here, ahead of the first stage, and parked in LDS behind the requests of
    // the first stages, in front of the first barrier (they arrive before the stage that barrier waits for anyway).
    // Written to LDS at this point they would hold the first wavefronts back for two trips to memory before their
    // share of the first stage is requested; fetched in the epilogue they are a trip that nothing covers.
    static_assert(kThreads >= BM && BM >= BN, "one thread per row scale");
    float cs_reg = 0.0f, bias_reg = 0.0f, rs_reg = 0.0f;
    if (Tile::kScaled) {
        if (tid < BN) {
            const int n = n0 + tid < N ? n0 + tid : N - 1;
            cs_reg = tile.cs[n];
            bias_reg = tile.bias ? tile.bias[n] : 0.0f;
        }
        if (tid < BM) rs_reg = tile.rs[m0 + tid < M ? m0 + tid : M - 1];
    }

    // wave-level load i of this wavefront fills rows (wave*6 + i)*8 .. +7 of the stage; lane l
    // fetches what belongs in slot l%8 of row l/8
    const int8_t* src[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int row = (wave * kLoads + i) * 8 + (lane >> 3);            // stage row 0..383
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        if (row < BM) {
            int gr = m0 + row;
            gr = gr < M ? gr : M - 1;
            src[i] = A + static_cast<size_t>(gr) * K + chunk * 16 + static_cast<size_t>(kt0) * kDmaRowBytes;
        } else {
            int gr = n0 + row - BM;
            gr = gr < N ? gr : N - 1;
            src[i] = W + static_cast<size_t>(gr) * K + chunk * 16 + static_cast<size_t>(kt0) * kDmaRowBytes;
        }
    }
    // loads FIRST, FIRST+1 of this wavefront's six
    auto issue_pair = [&](auto first, int kt, int slot) {
        constexpr int FIRST = decltype(first)::value;
        char* dst = lds_bytes + slot * kStageBytes + wave * (kLoads * 1024);
#pragma unroll
        for (int i = FIRST; i < FIRST + 2; ++i)
            __builtin_amdgcn_global_load_lds((global_void_ptr)(src[i] + static_cast<size_t>(kt) * kDmaRowBytes),
                                             (lds_void_ptr)(dst + i * 1024), 16, 0, 0);
    };
    auto issue = [&](int kt, int slot) {
        issue_pair(std::integral_constant<int, 0>{}, kt, slot);
        issue_pair(std::integral_constant<int, 2>{}, kt, slot);
        issue_pair(std::integral_constant<int, 4>{}, kt, slot);
        if constexpr (kLoads == 12) {
            issue_pair(std::integral_constant<int, 6>{}, kt, slot);
            issue_pair(std::integral_constant<int, 8>{}, kt, slot);
            issue_pair(std::integral_constant<int, 10>{}, kt, slot);
        }
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    // Fragment addresses.  Lane (row = lane % 32, half = lane / 32) of block i reads 16 bytes of
    // row base + 32 i, chunk 2 * substep + half.  All rows a lane touches differ by multiples of
    // 16, so they share one swizzle value, and the blocks are 32 rows = 4 KB apart: one address
    // register per operand and substep, the block picked by the instruction's offset field.
    const int frag_row = lane & 31, frag_half = lane >> 5;
    const uint32_t ring_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_ptr)ring));
    const uint32_t sw16 = ((frag_row >> 1) & 7) * 16;
    const uint32_t chunk_first = ((kh * 4 + frag_half) * 16) ^ sw16, chunk_second = ((kh * 4 + 2 + frag_half) * 16) ^ sw16;
    const uint32_t chunk_third = ((4 + frag_half) * 16) ^ sw16, chunk_fourth = ((6 + frag_half) * 16) ^ sw16;  // KSPLIT = 1
    const uint32_t a_row = ring_addr + (wm * WM + frag_row) * kDmaRowBytes;
    const uint32_t b_row = ring_addr + (BM + wn * WN + frag_row) * kDmaRowBytes;
    // the six reads of a substep, in two groups of three: (A0, A1, W0), then (W1, A2, A3)
    auto read_group = [&](auto group, int slot, uint32_t chunk_off, v4i (&fa)[TM], v4i (&fb)[TN]) {
        static_assert((TM == 4 || TM == 2) && TN == 2, "offsets below");
        const uint32_t a = a_row + slot * kStageBytes + chunk_off, b = b_row + slot * kStageBytes + chunk_off;
        if constexpr (TM == 2) {  // (A0, A1), then (W0, W1)
            if constexpr (decltype(group)::value == 0) {
                asm volatile("ds_read_b128 %0, %1" : "=v"(fa[0]) : "v"(a) : "memory");
                asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(fa[1]) : "v"(a) : "memory");
            } else {
                asm volatile("ds_read_b128 %0, %1" : "=v"(fb[0]) : "v"(b) : "memory");
                asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(fb[1]) : "v"(b) : "memory");
            }
        } else if constexpr (decltype(group)::value == 0) {
            asm volatile("ds_read_b128 %0, %1" : "=v"(fa[0]) : "v"(a) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(fa[1]) : "v"(a) : "memory");
            asm volatile("ds_read_b128 %0, %1" : "=v"(fb[0]) : "v"(b) : "memory");
        } else {
            asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(fb[1]) : "v"(b) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:8192" : "=v"(fa[2]) : "v"(a) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:12288" : "=v"(fa[3]) : "v"(a) : "memory");
        }
    };
    auto read_frags = [&](int slot, uint32_t chunk_off, v4i (&fa)[TM], v4i (&fb)[TN]) {
        read_group(std::integral_constant<int, 0>{}, slot, chunk_off, fa, fb);
        read_group(std::integral_constant<int, 1>{}, slot, chunk_off, fa, fb);
        // keep the reads ahead of the MFMAs that follow in program order: left alone, the
        // scheduler sinks them below those MFMAs to shorten the fragments' live ranges
        __builtin_amdgcn_sched_barrier(0);
    };
    // LDS reads of a wavefront return in order: once at most NEWER remain outstanding, every
    // read before the newest NEWER has delivered.  The fragments pass through the statement so
    // that the MFMAs consuming them cannot be moved above the wait.
    auto frags_ready = [&](auto newer, v4i (&fa)[TM], v4i (&fb)[TN]) {
        constexpr int kNewer = decltype(newer)::value;
        if constexpr (TM == 2) {
            asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]), "+v"(fb[1]) : "n"(kNewer));
        } else {
            asm volatile("s_waitcnt lgkmcnt(%6)"
                         : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1])
                         : "n"(kNewer));
        }
    };
    constexpr std::integral_constant<int, TM + TN> kOneBatch{};  // the reads of one substep
    constexpr std::integral_constant<int, 0> kNone{};
    // blocks i in [I0, I0 + 2); W fragment first: accumulator rows run along n
    auto multiply = [&](auto i0, const v4i (&fa)[TM], const v4i (&fb)[TN]) {
        constexpr int I0 = decltype(i0)::value;
#pragma unroll
        for (int i = I0; i < I0 + 2; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0);
    };
    constexpr std::integral_constant<int, 0> kLow{};
    constexpr std::integral_constant<int, 2> kHigh{};
    // one MFMA, block (I, J), fenced: nothing is scheduled across it
    auto multiply_one = [&](auto ic, auto jc, const v4i (&fa)[TM], const v4i (&fb)[TN]) {
        constexpr int I = decltype(ic)::value, J = decltype(jc)::value;
        __builtin_amdgcn_sched_barrier(0);
        acc[I][J] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[J], fa[I], acc[I][J], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    constexpr std::integral_constant<int, 0> k0{};
    constexpr std::integral_constant<int, 1> k1{};
    constexpr std::integral_constant<int, 2> k2{};
    constexpr std::integral_constant<int, 3> k3{};
    constexpr std::integral_constant<int, 4> k4{};
    constexpr std::integral_constant<int, 6> k6{};
    constexpr std::integral_constant<int, 8> k8{};
    constexpr std::integral_constant<int, 10> k10{};

#pragma unroll
    for (int s = 0; s < kDmaStages; ++s)
        if (s < nk) issue(s, s);
    TPQ_DMA_STAMP(1);
    if (Tile::kScaled) {  // behind the ring; read in the epilogue, many barriers later
        if (tid < BN) {
            cs_lds[tid] = cs_reg;
            cs_lds[BN + tid] = bias_reg;
        }
        if (tid < BM) rs_lds[tid] = rs_reg;
    }
    {  // this wavefront's share of stage 0: everything issued after it may still be outstanding
        const int younger = nk - 1 < kDmaStages - 1 ? nk - 1 : kDmaStages - 1;
        if (younger == 2) __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * kLoads));
        else if (younger == 1) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads));
        else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    }
    // The LDS counter is shared with scalar loads (kernel arguments, which return out of order)
    // and the column-scale writes above: drain it, so that only fragment reads are counted.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    TPQ_DMA_STAMP(2);

    v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
    int kt = 0, slot = 0;  // slot: kt % kDmaStages
    read_frags(0, chunk_first, fa0, fb0);
    if constexpr (KSPLIT == 0) {
    // Eight positions of 64 x 64, every wavefront multiplies all four substeps of a stage: no k-half exchange in the
    // epilogue, a third more fragment reads (four per four MFMAs).  The fragments of all four substeps are in
    // registers; the barrier stands in the middle of the stage, so that the requests for the next stage's first two
    // substeps have the MFMAs of two substeps to hide behind, as in the k-split form.
    v4i fa2[TM], fb2[TN], fa3[TM], fb3[TN];
    constexpr std::integral_constant<int, 3 * (TM + TN)> kThreeBatches{};
    constexpr std::integral_constant<int, 2 * (TM + TN)> kTwoBatches{};
    read_frags(0, chunk_second, fa1, fb1);
    for (; kt + kDmaStages < nk; ++kt) {  // steady state: stages kt+1 .. kt+3 all exist
        const int next = slot == kDmaStages - 1 ? 0 : slot + 1;
        read_frags(slot, chunk_third, fa2, fb2);
        read_frags(slot, chunk_fourth, fa3, fb3);
        frags_ready(kThreeBatches, fa0, fb0);
        multiply(kLow, fa0, fb0);
        frags_ready(kTwoBatches, fa1, fb1);
        multiply(kLow, fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        frags_ready(kNone, fa2, fb2);  // this wavefront is done reading stage kt
        frags_ready(kNone, fa3, fb3);
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads));
        asm volatile("s_barrier" ::: "memory");
        multiply_one(k0, k0, fa2, fb2);
        read_group(k0, next, chunk_first, fa0, fb0);
        multiply_one(k0, k1, fa2, fb2);
        read_group(k1, next, chunk_first, fa0, fb0);
        multiply_one(k1, k0, fa2, fb2);
        read_group(k0, next, chunk_second, fa1, fb1);
        multiply_one(k1, k1, fa2, fb2);
        read_group(k1, next, chunk_second, fa1, fb1);
        multiply_one(k0, k0, fa3, fb3);
        issue_pair(k0, kt + kDmaStages, slot);
        multiply_one(k0, k1, fa3, fb3);
        issue_pair(k2, kt + kDmaStages, slot);
        multiply_one(k1, k0, fa3, fb3);
        issue_pair(k4, kt + kDmaStages, slot);
        multiply_one(k1, k1, fa3, fb3);
        slot = next;
    }
    for (; kt < nk; ++kt) {  // last stages: nothing left to issue
        const int next = slot == kDmaStages - 1 ? 0 : slot + 1;
        read_frags(slot, chunk_third, fa2, fb2);
        read_frags(slot, chunk_fourth, fa3, fb3);
        frags_ready(kThreeBatches, fa0, fb0);
        multiply(kLow, fa0, fb0);
        frags_ready(kTwoBatches, fa1, fb1);
        multiply(kLow, fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        frags_ready(kNone, fa2, fb2);
        frags_ready(kNone, fa3, fb3);
        if (kt + 1 < nk) {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            asm volatile("s_barrier" ::: "memory");
            read_frags(next, chunk_first, fa0, fb0);
            read_frags(next, chunk_second, fa1, fb1);
        }
        multiply(kLow, fa2, fb2);
        multiply(kLow, fa3, fb3);
        slot = next;
    }
    } else if constexpr (KSPLIT == 1) {
    for (; kt + kDmaStages < nk; ++kt) {  // steady state: stages kt+1 .. kt+3 all exist
        const int next = slot == kDmaStages - 1 ? 0 : slot + 1;
        read_frags(slot, chunk_second, fa1, fb1);
        frags_ready(kOneBatch, fa0, fb0);
        multiply(kLow, fa0, fb0);
        multiply(kHigh, fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot, chunk_third, fa0, fb0);
        frags_ready(kOneBatch, fa1, fb1);
        multiply(kLow, fa1, fb1);
        multiply(kHigh, fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot, chunk_fourth, fa1, fb1);
        frags_ready(kOneBatch, fa0, fb0);
        multiply(kLow, fa0, fb0);
        multiply(kHigh, fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        frags_ready(kNone, fa1, fb1);  // this wavefront is done reading stage kt
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads));
        asm volatile("s_barrier" ::: "memory");
        multiply_one(k0, k0, fa1, fb1);
        read_group(k0, next, chunk_first, fa0, fb0);
        multiply_one(k0, k1, fa1, fb1);
        read_group(k1, next, chunk_first, fa0, fb0);
        multiply_one(k1, k0, fa1, fb1);
        issue_pair(k0, kt + kDmaStages, slot);
        multiply_one(k1, k1, fa1, fb1);
        issue_pair(k2, kt + kDmaStages, slot);
        multiply_one(k2, k0, fa1, fb1);
        issue_pair(k4, kt + kDmaStages, slot);
        multiply_one(k2, k1, fa1, fb1);
        if constexpr (kLoads == 12) issue_pair(k6, kt + kDmaStages, slot);
        multiply_one(k3, k0, fa1, fb1);
        if constexpr (kLoads == 12) issue_pair(k8, kt + kDmaStages, slot);
        multiply_one(k3, k1, fa1, fb1);
        if constexpr (kLoads == 12) issue_pair(k10, kt + kDmaStages, slot);
        slot = next;
    }
    for (; kt < nk; ++kt) {  // last stages: nothing left to issue
        const int next = slot == kDmaStages - 1 ? 0 : slot + 1;
        read_frags(slot, chunk_second, fa1, fb1);
        frags_ready(kOneBatch, fa0, fb0);
        multiply(kLow, fa0, fb0);
        multiply(kHigh, fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot, chunk_third, fa0, fb0);
        frags_ready(kOneBatch, fa1, fb1);
        multiply(kLow, fa1, fb1);
        multiply(kHigh, fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot, chunk_fourth, fa1, fb1);
        frags_ready(kOneBatch, fa0, fb0);
        multiply(kLow, fa0, fb0);
        multiply(kHigh, fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        frags_ready(kNone, fa1, fb1);
        if (kt + 1 < nk) {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            asm volatile("s_barrier" ::: "memory");
            read_frags(next, chunk_first, fa0, fb0);
        }
        multiply(kLow, fa1, fb1);
        multiply(kHigh, fa1, fb1);
        slot = next;
    }
    } else {
    for (; kt + kDmaStages < nk; ++kt) {  // steady state: stages kt+1 .. kt+3 all exist
        const int next = slot == kDmaStages - 1 ? 0 : slot + 1;
        read_frags(slot, chunk_second, fa1, fb1);
        frags_ready(kOneBatch, fa0, fb0);
        multiply(kLow, fa0, fb0);
        multiply(kHigh, fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);  // the waits below stay behind the MFMAs that cover them
        frags_ready(kNone, fa1, fb1);  // this wavefront is done reading stage kt
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads));  // own share of kt+1 landed (kt+2 may be in flight)
        asm volatile("s_barrier" ::: "memory");
        // Second substep.  An MFMA occupies the matrix core for 32 clocks but the wavefront's
        // issue slot only briefly, so the fragment requests for stage kt+1 and the refill (address
        // arithmetic and all) go between the MFMAs instead of in front of them.
        multiply_one(k0, k0, fa1, fb1);
        read_group(k0, next, chunk_first, fa0, fb0);
        multiply_one(k0, k1, fa1, fb1);
        read_group(k1, next, chunk_first, fa0, fb0);
        multiply_one(k1, k0, fa1, fb1);
        issue_pair(k0, kt + kDmaStages, slot);
        multiply_one(k1, k1, fa1, fb1);
        issue_pair(k2, kt + kDmaStages, slot);
        multiply_one(k2, k0, fa1, fb1);
        issue_pair(k4, kt + kDmaStages, slot);
        multiply_one(k2, k1, fa1, fb1);
        multiply_one(k3, k0, fa1, fb1);
        multiply_one(k3, k1, fa1, fb1);
        slot = next;
    }
    for (; kt < nk; ++kt) {  // last stages: nothing left to issue
        const int next = slot == kDmaStages - 1 ? 0 : slot + 1;
        read_frags(slot, chunk_second, fa1, fb1);
        frags_ready(kOneBatch, fa0, fb0);
        multiply(kLow, fa0, fb0);
        multiply(kHigh, fa0, fb0);
        frags_ready(kNone, fa1, fb1);
        if (kt + 1 < nk) {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            asm volatile("s_barrier" ::: "memory");
            read_frags(next, chunk_first, fa0, fb0);
        }
        multiply(kLow, fa1, fb1);
        multiply(kHigh, fa1, fb1);
        slot = next;
    }

    }

    // ---- epilogue ------------------------------------------------------------------------------------
    TPQ_DMA_STAMP(3);
    const bool has_bias = tile.bias != nullptr;
    if constexpr (KSPLIT == 0) if ((vector_stores & 2) == 0) {
        // Every wavefront finishes its own 64 x 64 block, without a barrier: the two stage buffers that do not hold
        // the last stage are free since the last barrier of the main loop (every wavefront had finished reading them
        // and every direct load had landed), so each wavefront turns its block into row order in 12 KB of its own
        // there and stores it itself, 16 bytes per lane, whole 128-byte lines.  16-bit outputs: all 64 rows at once;
        // 32-bit outputs (the partial sums of a sliced launch, float32): two passes of 32 rows through the same 12 KB.
        const int last = slot == 0 ? kDmaStages - 1 : slot - 1;  // buffer of the last stage (slot was advanced past it)
        const int mine = wave < 4 ? (last == 0 ? 1 : 0) : (last == 2 ? 1 : 2);
        constexpr int kElem = sizeof(out_t);
        constexpr int kPassBlocks = kElem == 2 ? TM : 1;             // 32-row blocks per pass
        constexpr int kWavePitch = WN * kElem + 16;                  // bytes per row of the wavefront's image
        constexpr int kRowChunks = WN * kElem / 16;                  // 16-byte chunks per row: 8 or 16
        constexpr int kRowsPerStore = kWave / kRowChunks;            // rows per wavefront store: 8 or 4
        static_assert(4 * 12288 <= kStageBytes && kPassBlocks * 32 * kWavePitch <= 12288, "four wavefronts per free buffer");
        char* img = lds_bytes + mine * kStageBytes + (wave & 3) * 12288;
#pragma unroll
        for (int first = 0; first < TM; first += kPassBlocks) {
            float rs_r[kPassBlocks];
#pragma unroll
            for (int i = 0; i < kPassBlocks; ++i) rs_r[i] = Tile::kScaled ? rs_lds[wm * WM + (first + i) * 32 + frag_row] : 0.0f;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n_wave = j * 32 + 8 * q + 4 * frag_half;  // 4 consecutive columns of the wavefront's 64
                    float c4[4] = {0, 0, 0, 0}, b4[4] = {0, 0, 0, 0};
                    if (Tile::kScaled) {
                        const float4 c = *reinterpret_cast<const float4*>(cs_lds + wn * WN + n_wave);
                        const float4 b = *reinterpret_cast<const float4*>(cs_lds + BN + wn * WN + n_wave);
                        c4[0] = c.x; c4[1] = c.y; c4[2] = c.z; c4[3] = c.w;
                        b4[0] = b.x; b4[1] = b.y; b4[2] = b.z; b4[3] = b.w;
                    }
#pragma unroll
                    for (int i = 0; i < kPassBlocks; ++i) {
                        char* dst = img + (i * 32 + frag_row) * kWavePitch + n_wave * kElem;
                        if constexpr (kElem == 2) {
                            float f[4];
#pragma unroll
                            for (int t = 0; t < 4; ++t) f[t] = Tile::value(acc[first + i][j][4 * q + t], rs_r[i], c4[t], b4[t], has_bias);
                            *reinterpret_cast<uint2*>(dst) = make_uint2(Tile::pack2(f[0], f[1]), Tile::pack2(f[2], f[3]));
                        } else {
                            out_t vals[4];
#pragma unroll
                            for (int t = 0; t < 4; ++t) vals[t] = Tile::convert(acc[first + i][j][4 * q + t], rs_r[i], c4[t], b4[t], has_bias);
                            *reinterpret_cast<uint4*>(dst) = make_uint4(__builtin_bit_cast(uint32_t, vals[0]), __builtin_bit_cast(uint32_t, vals[1]),
                                                                        __builtin_bit_cast(uint32_t, vals[2]), __builtin_bit_cast(uint32_t, vals[3]));
                        }
                    }
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wavefront's own LDS writes, in order with its reads
            if (first == 0) TPQ_DMA_STAMP(5);
#pragma unroll
            for (int it = 0; it < kPassBlocks * 32 / kRowsPerStore; ++it) {
                const int row = it * kRowsPerStore + lane / kRowChunks, col = (lane % kRowChunks) * (16 / kElem);
                const int m = m0 + wm * WM + first * 32 + row, n = n0 + wn * WN + col;
                const uint4 v = *reinterpret_cast<const uint4*>(img + row * kWavePitch + col * kElem);
                if (m >= M || n >= N) continue;
                out_t* dstp = tile.out + (static_cast<size_t>(blockIdx.y) * M + m) * N + n;
                if ((vector_stores & 1) && n + 16 / kElem <= N) {
                    nt_store(reinterpret_cast<uint4*>(dstp), v);  // written once, read by a later kernel
                } else {
                    const uint32_t words[4] = {v.x, v.y, v.z, v.w};
                    if constexpr (kElem == 2) {
                        for (int e = 0; e < 8 && n + e < N; ++e) dstp[e] = static_cast<out_t>(words[e >> 1] >> (16 * (e & 1)));
                    } else {
                        for (int e = 0; e < 4 && n + e < N; ++e) dstp[e] = __builtin_bit_cast(out_t, words[e]);
                    }
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the image has been read before the next pass overwrites it
        }
        TPQ_DMA_STAMP(6);
        return;
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // ring no longer needed
    // Exchange: a wavefront keeps blocks i in [KEEP, KEEP+2) and hands the other two to its
    // partner (same position, other k-half), 16 KB per wavefront.
    int4* mine = reinterpret_cast<int4*>(lds_bytes) + wave * (16 * kWave) + lane;
    const int4* theirs = reinterpret_cast<const int4*>(lds_bytes) + (wave ^ 4) * (16 * kWave) + lane;
    auto hand_over = [&](auto give) {
        constexpr int G = decltype(give)::value;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    mine[((i * TN + j) * 4 + q) * kWave] = make_int4(acc[G + i][j][4 * q], acc[G + i][j][4 * q + 1],
                                                                     acc[G + i][j][4 * q + 2], acc[G + i][j][4 * q + 3]);
    };
    auto take_over = [&](auto keep) {
        constexpr int KEEP = decltype(keep)::value;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int4 o = theirs[((i * TN + j) * 4 + q) * kWave];
                    acc[KEEP + i][j][4 * q] += o.x; acc[KEEP + i][j][4 * q + 1] += o.y;
                    acc[KEEP + i][j][4 * q + 2] += o.z; acc[KEEP + i][j][4 * q + 3] += o.w;
                }
    };
    // scale, convert and place blocks [KEEP, KEEP+2) in the image
    auto to_image = [&](auto keep) {
        constexpr int KEEP = decltype(keep)::value;
        float rs_r[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            rs_r[i] = Tile::kScaled ? rs_lds[wm * WM + (KEEP + i) * 32 + frag_row] : 0.0f;
        }
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
                for (int i = 0; i < 2; ++i) {
                    const int m_local = wm * WM + (KEEP + i) * 32 + frag_row;
                    char* dst = lds_bytes + m_local * kPitch + n_local * sizeof(out_t);
                    if constexpr (sizeof(out_t) == 2) {
                        float f[4];
#pragma unroll
                        for (int t = 0; t < 4; ++t) f[t] = Tile::value(acc[KEEP + i][j][4 * q + t], rs_r[i], c4[t], b4[t], has_bias);
                        *reinterpret_cast<uint2*>(dst) = make_uint2(Tile::pack2(f[0], f[1]), Tile::pack2(f[2], f[3]));
                    } else {
                        out_t vals[4];
#pragma unroll
                        for (int t = 0; t < 4; ++t) vals[t] = Tile::convert(acc[KEEP + i][j][4 * q + t], rs_r[i], c4[t], b4[t], has_bias);
                        *reinterpret_cast<uint4*>(dst) = make_uint4(__builtin_bit_cast(uint32_t, vals[0]), __builtin_bit_cast(uint32_t, vals[1]),
                                                                    __builtin_bit_cast(uint32_t, vals[2]), __builtin_bit_cast(uint32_t, vals[3]));
                    }
                }
            }
    };
    if constexpr (KSPLIT == 2) {
        if (kh == 0) hand_over(kHigh); else hand_over(kLow);
        __syncthreads();
        if (kh == 0) take_over(kLow); else take_over(kHigh);
        __syncthreads();  // exchange area consumed before the image overwrites it
        TPQ_DMA_STAMP(4);
        if (kh == 0) to_image(kLow); else to_image(kHigh);
    } else {
        to_image(kLow);
        if constexpr (TM == 4) to_image(kHigh);
    }
    __syncthreads();
    TPQ_DMA_STAMP(5);
    constexpr int kChunksPerOutRow = BN / kPerChunk;  // 16-byte chunks per image row
    for (int c = tid; c < BM * kChunksPerOutRow; c += kThreads) {
        const int row = c / kChunksPerOutRow, col = (c % kChunksPerOutRow) * kPerChunk;
        const int m = m0 + row, n = n0 + col;
        if (m >= M || n >= N) continue;
        const char* srcp = lds_bytes + row * kPitch + col * sizeof(out_t);
        out_t* dstp = tile.out + (static_cast<size_t>(blockIdx.y) * M + m) * N + n;
        if ((vector_stores & 1) && n + kPerChunk <= N) {
            nt_store(reinterpret_cast<uint4*>(dstp), *reinterpret_cast<const uint4*>(srcp));  // written once, read by a later kernel
        } else {
            for (int e = 0; e < kPerChunk && n + e < N; ++e) dstp[e] = reinterpret_cast<const out_t*>(srcp)[e];
        }
    }
    TPQ_DMA_STAMP(6);
}

// K must be a multiple of the 128-byte stage.
// Up to 128 rows the 256-row tiles are half empty: worth it only where N alone yields tiles for the whole chip.
inline bool dma_path_ok(int64_t M, int64_t N, int64_t K) { return (M > 128 || (M > 32 && N >= 16384)) && K % kDmaRowBytes == 0; }

template <int KSPLIT, class Tile>
int launch_dma_split(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Tile tile, hipStream_t s, int slices = 1) {
    constexpr size_t smem = static_cast<size_t>(kDmaStages) * (256 + 128) * kDmaRowBytes + (2 * 128 + 256) * sizeof(float);
    const int64_t tiles = ((M + 255) / 256) * ((N + 127) / 128);
    TPQ_REQUIRE(tiles <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "int8 gemm: too many tiles");
    auto kernel = int8_gemm_dma_kernel<Tile, KSPLIT>;
    static std::atomic<uint64_t> configured{0};  // per instantiation
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), smem, configured, "int8 gemm")) return rc;
    int vector_stores = (N * sizeof(typename Tile::out_t)) % 16 == 0 && aligned(tile.out, 16);
    if (tuning_env("TPQ_INT8_NO_WAVE_EPILOGUE")) vector_stores |= 2;  // comparison runs: the workgroup-wide epilogue
    kernel<<<dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(slices)), KSPLIT == 1 ? 256 : 512, smem, s>>>(
        a, w, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), tile, vector_stores, slices);
    return check_launch("int8 mfma gemm (dma)");
}

// Which form of the kernel.  Eight positions without a k split (0) save the exchange of the k-halves in the epilogue
// (5,100 of a workgroup's 62,700 clocks at 2048 x 4096 x 4096) and pay a third more fragment reads per stage: measured
// against the k-split form (2) with the same result bits: 2048 x 4096 x 4096 -2 %, K = 2048 -6 %, 2048 x 6912 x 2560
// -4 %, the sliced launches at 128 .. 1024 rows of 4096 x 4096 -4 .. -7.5 %, 256 x 8192 x 8192 (sliced) -2 %; from 64
// stages per workgroup on the k-split form is as fast or faster (2048 x 4096 x 11008 +0.6 %, 300 x 28672 x 8192 +1.4 %,
// 8192^3 +0.6 % for the eight positions), so it keeps those.  TPQ_INT8_KSPLIT = 0 / 1 / 2 in a tuning build forces a
// form (1: four wavefronts, no k split, 128 x 64 per wavefront).
template <class Tile>
int launch_dma(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Tile tile, hipStream_t s, int slices = 1) {
    const char* env = tuning_env("TPQ_INT8_KSPLIT");
    if (env && env[0] == '1') return launch_dma_split<1>(a, w, M, N, K, tile, s, slices);
    if (env && env[0] == '0') return launch_dma_split<0>(a, w, M, N, K, tile, s, slices);
    if (env && env[0] == '2') return launch_dma_split<2>(a, w, M, N, K, tile, s, slices);
    const int64_t stages = K / kDmaRowBytes, per_workgroup = (stages + slices - 1) / slices;
    if (per_workgroup < 64) return launch_dma_split<0>(a, w, M, N, K, tile, s, slices);
    return launch_dma_split<2>(a, w, M, N, K, tile, s, slices);
}

// Few output tiles and a long k range (a few hundred rows against a square weight): each tile's k range is cut
// into slices of whole stages, one workgroup per slice, each writing its exact partial sums to a matrix of its
// own; a second kernel adds them.  How many slices: enough workgroups for the chip, at least four stages each
// and none empty; 1 = not worth it.
inline int dma_slices(int64_t M, int64_t N, int64_t K) {
    static const int forced = [] { const char* e = tuning_env("TPQ_INT8_SLICES"); return e ? std::atoi(e) : 0; }();
    if (M < 1 || K % kDmaRowBytes != 0) return 1;
    const int64_t tiles = ((M + 255) / 256) * ((N + 127) / 128), nk = K / kDmaRowBytes;
    static const int min_stages = [] { const char* e = tuning_env("TPQ_INT8_SLICE_STAGES"); return e ? std::atoi(e) : 4; }();
    static const int target = [] { const char* e = tuning_env("TPQ_INT8_SLICE_TARGET"); return e ? std::atoi(e) : 256; }();
    int64_t slices = forced ? forced : target / tiles;
    if (slices > nk / min_stages) slices = nk / min_stages;
    if (slices < 2) return 1;
    const int64_t per = (nk + slices - 1) / slices;
    return static_cast<int>((nk + per - 1) / per);  // drop slices that would start past the end
}

// partial [slices][M][N] int32 (16-byte aligned) := the slices of A W^T
inline int launch_dma_sliced(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, int32_t* partial, int slices, hipStream_t s) {
    const TileInt32 tile{partial, nullptr, nullptr, nullptr};
    return launch_dma(a, w, M, N, K, tile, s, slices);
}

}  // namespace
}  // namespace tpq
