// Tiled GEMM C = A W^T (int8 -> int32, or float16 / bfloat16 -> float32), staggered form: 256 x 128 tile per workgroup,
// three-stage LDS ring of whole 128-byte rows filled by direct global -> LDS loads, eight wavefronts in eight positions of 64 x 64 (v_mfma_i32_16x16x64_i8), the two
// wavefronts of a SIMD half a stage apart.
//
// What the form answers (measured on MI355X at 2048 x 4096 x 4096, per stage of 128 bytes of k and compute unit): the
// matrix cores need 1024 - 1090 clocks, the vector memory path 1040 (48 wave-level loads of 1 KB, one per ~21.6
// clocks), so both have to run all the time; the lock-step kernel (int8_gemm_dma.h) took 1450 - 1490.  Found:
//  (i)   A SIMD issues matrix and vector ALU instructions through one port, older wavefront first.  While one
//        wavefront issues MFMAs back to back, every vector instruction of another one (the address arithmetic of a
//        fragment read or of a direct load) waits for a gap; a wavefront that mixes them with its own MFMAs delays
//        those.  (Two loading wavefronts beside two multiplying ones on a SIMD: the MFMAs kept their rate, the loads
//        dropped to a third of theirs.)
//  (ii)  A direct load blocks the wavefront that issues it until the memory path accepts it, and with it every MFMA
//        behind it in program order.
//  (iii) The chip runs this kernel at its power limit (random operands: 1.4 - 1.7 GHz of 2.4), so time follows energy
//        more than clocks.  v_mfma_i32_16x16x64_i8 reads and writes a quarter of the accumulator registers of
//        v_mfma_i32_32x32x32_i8 per multiply-add and sustains 4.1 POPS alone where that one sustains 3.5.
// So:
//   - a wavefront alternates between a multiply phase (the 32 MFMAs of a stage, all fragments already in registers,
//     nothing else) and a memory phase (the 16 fragment reads of its next stage and its six direct loads), with a
//     workgroup barrier at the end of every phase; wavefronts 0..3 multiply in the even phases, 4..7 in the odd ones,
//     so every SIMD always has one wavefront whose MFMAs wait for nothing.  (One barrier per stage and no forced
//     alternation was measured too: the multiply phases of a SIMD's two wavefronts drift together, + 4 %.)
//   - the memory phase contains no vector ALU instruction: fragment addresses are 12 registers computed once (per
//     ring slot, operand and k-half; the loop is unrolled three times so that the slot is a constant), and the
//     direct loads take a scalar base (advanced per stage by scalar instructions) plus a per-lane 32-bit offset that
//     never changes.  The loads are spread between the reads, so the memory path has work from the start of a phase.
//
// Ring protocol for a ring of S stages (S = 3; stage t lives in slot t % S; the prologue requests stages 0 .. S - 2 and
// group 0's share of stage S - 1).  Group 0 reads stage t in phase 2t - 1,
// group 1 in phase 2t; the barrier that ends phase 2t frees the slot.  Every wavefront requests its eighth of a stage in
// its own memory phase: group 0 requests stage t + S in phase 2t + 1, group 1 requests stage t + S - 1 in phase 2t (into
// the slot of stage t - 1).  A stage must have landed when the barrier that ends phase 2t - 2 is crossed; each wavefront
// waits for its own share in front of that barrier (vector loads of a wavefront complete in order, so "my share of
// t + 1 has landed" is "at most the loads of the S - 2 stages behind it are outstanding").  Both groups cross 2 nk - 1
// barriers after the first.  A fourth stage for the 128-row tile (128 KB of LDS) was measured where the weight streams
// from HBM and a compute unit pulls about 25 GB/s of it: no change (4096 x 4096 at 256 .. 1024 rows 21.1 .. 22.5 us
// against 21.4 .. 22.6), so that rate is not set by the depth of the ring.
//
// Four extra wavefronts that do nothing but request (one per SIMD, 168 registers per wavefront) were built and measured:
// the loop drops from 1085 to 1064 clocks per stage, the first stage arrives 1000 clocks later, same time; not kept.
//
// Requires K % 128 == 0, K < 2^23 and 16-byte aligned operands.  Edges in M and N: source rows are clamped, stores masked.
#pragma once

#include "int8_gemm_dma.h"

namespace tpq {
namespace {

#ifndef TPQ_PHASE_PRIO
#define TPQ_PHASE_PRIO 1
#endif
constexpr int kPhasePrio = TPQ_PHASE_PRIO;  // wavefront priority during a multiply phase

#if defined(TPQ_DMA_STAMPS) && TPQ_DMA_STAMPS >= 2
#define TPQ_STAGGER_PHASE_STAMPS 1
__device__ unsigned long long g_stagger_stamps[8 * 128];  // [wavefront][phase][arrival at the barrier, departure]
constexpr int kStaggerStampBytes = 8 * 128 * 8;
#else
constexpr int kStaggerStampBytes = 0;
#endif
#ifdef TPQ_DMA_STAMPS
__device__ unsigned long long g_stagger_coarse[4 * 8];  // [start, first barrier crossed, main loop done, end][wavefront], one workgroup
#define TPQ_STAGGER_STAMP(I) do { if (blockIdx.x == 9 && wave < 8 && lane == 0) g_stagger_coarse[(I) * 8 + wave] = __builtin_amdgcn_s_memtime(); } while (0)
#else
#define TPQ_STAGGER_STAMP(I) do { } while (0)
#endif

typedef float v4f __attribute__((ext_vector_type(4)));

// f(integral_constant<int, I>) for I = FIRST .. LAST - 1, unrolled at compile time
template <int FIRST, int LAST, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>{});
        static_for<FIRST + 1, LAST>(f);
    }
}
// if (base + 0 < limit) { f(0); if (base + 1 < limit) { f(1); ... } }: up to DEPTH steps as nested straight-line code
template <int D, int DEPTH, class F>
__device__ __forceinline__ void nested_while_below(int base, int limit, F&& f) {
    if constexpr (D < DEPTH) {
        if (base + D < limit) {
            f(std::integral_constant<int, D>{});
            nested_while_below<D + 1, DEPTH>(base, limit, f);
        }
    }
}

// The operand types the form multiplies.  A stage is 128 bytes of k per row whatever the type, and the lane layout of
// the 16-byte fragments is the same for all three instructions (lane (r, c): row r, bytes 16 c .. 16 c + 15 of a k-half
// of 64 bytes), so the kernel body does not depend on the type beyond the accumulator and the instruction.
struct ArithI8 {  // 128 k per stage, v_mfma_i32_16x16x64_i8
    using acc_t = v4i;
    static __device__ __forceinline__ acc_t mfma(const v4i& b, const v4i& a, const acc_t& c) { return __builtin_amdgcn_mfma_i32_16x16x64_i8(b, a, c, 0, 0, 0); }
};
struct ArithF16 {  // 64 k per stage, v_mfma_f32_16x16x32_f16
    using acc_t = v4f;
    static __device__ __forceinline__ acc_t mfma(const v4i& b, const v4i& a, const acc_t& c) {
        typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8_t, b), __builtin_bit_cast(h8_t, a), c, 0, 0, 0);
    }
};
struct ArithBF16 {  // 64 k per stage, v_mfma_f32_16x16x32_bf16
    using acc_t = v4f;
    static __device__ __forceinline__ acc_t mfma(const v4i& b, const v4i& a, const acc_t& c) {
        typedef __bf16 b8_t __attribute__((ext_vector_type(8)));
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8_t, b), __builtin_bit_cast(b8_t, a), c, 0, 0, 0);
    }
};
struct ArithF32 {  // 32 k per stage, four v_mfma_f32_16x16x4_f32 per fragment: float t of every lane's four is k = 4 c + t
    using acc_t = v4f;
    static __device__ __forceinline__ acc_t mfma(const v4i& b, const v4i& a, const acc_t& c) {
        const v4f bf = __builtin_bit_cast(v4f, b), af = __builtin_bit_cast(v4f, a);
        acc_t d = __builtin_amdgcn_mfma_f32_16x16x4f32(bf.x, af.x, c, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(bf.y, af.y, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(bf.z, af.z, d, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_16x16x4f32(bf.w, af.w, d, 0, 0, 0);
    }
};

// A, W: row-major [M][K], [N][K] with K contiguous; row_bytes = K * sizeof(element).
// MB: blocks of 16 rows per wavefront: 4 (tile of 256 rows, what the description above and the numbers are about) or 2
// (tile of 128 rows for problems with few rows or few tiles: per stage 32 wave-level loads against 16 MFMAs per
// wavefront, so the vector memory path bounds it at about 700 clocks per stage; int8, 4096 x 4096: 15.4 .. 18.8 us at
// 256 .. 1024 rows, where the 256-row tiles take 21 .. 22 and the sliced launches 21 .. 32).
template <class Tile, class Arith, int MB>
__global__ __launch_bounds__(512) void gemm_stagger_kernel(const char* __restrict__ A, const char* __restrict__ W, int M, int N,
                                                                         int row_bytes, Tile tile, int vector_stores, int slices) {
    using out_t = typename Tile::out_t;
    using acc_t = typename Arith::acc_t;
    constexpr int BM = 64 * MB, BN = 128, WM = 16 * MB, WN = 64;
    static_assert(MB == 4 || MB == 2, "two tile heights are built");
    constexpr int kStageBytes = (BM + BN) * kDmaRowBytes;  // 48 KB (32 KB)
    constexpr int S = kDmaStages;                          // ring depth (the loop control below is written for any depth >= 3)
    constexpr int kRingBytes = S * kStageBytes;            // 144 KB (96 KB)
    constexpr int kRequesters = 8;
    constexpr int kLoadsA = BM / 8 / kRequesters, kLoadsW = BN / 8 / kRequesters, kLoads = kLoadsA + kLoadsW;  // 4 + 2
    extern __shared__ uint4 ring[];
    char* lds_bytes = reinterpret_cast<char*>(ring);
    float* cs_lds = reinterpret_cast<float*>(lds_bytes + kRingBytes);  // [BN] column scales, [BN] bias, [BM] row scales
    float* rs_lds = cs_lds + 2 * BN;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (wave >> 1) & 3, wn = wave & 1;
    TPQ_STAGGER_STAMP(0);

    // tile of this workgroup: every XCD (workgroup id mod 8) gets a compact patch of tiles, see int8_gemm_dma_kernel
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tile_m, tile_n;
    {
        const int id = blockIdx.x, total = tiles_m * tiles_n;
        if (total % 8 == 0 && tiles_m % 2 == 0 && tiles_n % 4 == 0) {
            const int xcd = id & 7, local = id >> 3;
            const int pm = tiles_m / 2, pn = tiles_n / 4;
            tile_m = (xcd & 1) * pm + local % pm;
            tile_n = (xcd >> 1) * pn + local / pm;
        } else {
            tile_m = id % tiles_m;
            tile_n = id / tiles_m;
        }
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int nk_all = row_bytes / kDmaRowBytes, nk_slice = (nk_all + slices - 1) / slices;
    const int kt0 = blockIdx.y * nk_slice;
    const int nk = nk_all - kt0 < nk_slice ? nk_all - kt0 : nk_slice;

    // ---- requests -----------------------------------------------------------------------------------------------
    // Wavefront r owns row blocks of eight rows: kLoadsA of the activations, kLoadsW of
    // the weights.  Load i of a requester fills 1 KB of the stage: lane l fetches the 16-byte chunk that belongs in
    // slot l % 8 of row l / 8 (the swizzle of the fragment reads is applied on the global side).
    const int rq = wave;
    uint32_t voff[kLoads];            // byte offset of this lane's chunk from the tile's first row, k = 0
    uint32_t lds_of_load[kLoads];     // byte offset of the load's 1 KB inside a stage (wave-uniform)
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const bool act = i < kLoadsA;
        const int block = act ? rq * kLoadsA + i : rq * kLoadsW + (i - kLoadsA);  // block of eight rows inside the operand's tile
        const int row = block * 8 + (lane >> 3);                                 // row inside the operand's tile
        const int stage_row = act ? row : BM + row;
        const int chunk = (lane & 7) ^ ((stage_row >> 1) & 7);
        int gr = (act ? m0 : n0) + row;
        const int limit = act ? M : N;
        gr = gr < limit ? gr : limit - 1;
        voff[i] = static_cast<uint32_t>(gr - (act ? m0 : n0)) * static_cast<uint32_t>(row_bytes) + chunk * 16;
        lds_of_load[i] = static_cast<uint32_t>(act ? block : BM / 8 + block) * 1024;
    }
    const uint32_t ring_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_ptr)ring));
    const char* const base_a = A + static_cast<size_t>(m0) * row_bytes + static_cast<size_t>(kt0) * kDmaRowBytes;
    const char* const base_w = W + static_cast<size_t>(n0) * row_bytes + static_cast<size_t>(kt0) * kDmaRowBytes;
    // loads [FIRST, FIRST + COUNT) of stage kt into ring slot SLOT: scalar base, constant per-lane offset, no vector ALU
    auto request = [&](auto first, auto count, auto slot_c, int kt) {
        constexpr int FIRST = decltype(first)::value, COUNT = decltype(count)::value, SLOT = decltype(slot_c)::value;
        const char* const sa = base_a + static_cast<size_t>(kt) * kDmaRowBytes;
        const char* const sw = base_w + static_cast<size_t>(kt) * kDmaRowBytes;
#pragma unroll
        for (int i = FIRST; i < FIRST + COUNT; ++i) {
            const uint32_t dst = ring_addr + SLOT * kStageBytes + lds_of_load[i];
            const uint32_t off = voff[i];
            if (i < kLoadsA) {
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(sa) : "memory", "m0");
            } else {
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(sw) : "memory", "m0");
            }
        }
    };
    constexpr std::integral_constant<int, 0> c0{};
    constexpr std::integral_constant<int, kLoads> cAll{};
        auto request_stage = [&](auto slot_c, int kt) { request(c0, cAll, slot_c, kt); };

    // ---- fragment reads -----------------------------------------------------------------------------------------
    // v_mfma_i32_16x16x64_i8: lane (r = lane % 16, c = lane / 16) holds row r, 16-byte chunk c of a k-half of 64 bytes.
    // (On random operands at the power limit this shape sustains 4.1 POPS where 32x32x32 sustains 3.5: a quarter of the
    // accumulator registers read and written per multiply-add.)  One address register per ring slot, operand and
    // k-half; the four blocks of 16 rows are the instruction's offset.  Rows a lane touches differ by multiples of 16, so
    // they share one swizzle value.
    const int frag_row = lane & 15, frag_chunk = lane >> 4;
    const uint32_t sw = (frag_row >> 1) & 7;
    uint32_t addr_a[S][2], addr_b[S][2];
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
            const uint32_t chunk = ((kh * 4 + frag_chunk) ^ sw) * 16;
            addr_a[s][kh] = ring_addr + s * kStageBytes + (wm * WM + frag_row) * kDmaRowBytes + chunk;
            addr_b[s][kh] = ring_addr + s * kStageBytes + (BM + wn * WN + frag_row) * kDmaRowBytes + chunk;
        }
    v4i fa[2][MB], fb[2][4];  // [k-half][block of 16 rows]
    auto read_half = [&](auto slot_c, auto half_c) {
        constexpr int SLOT = decltype(slot_c)::value;
#pragma unroll
        for (int kh = decltype(half_c)::value; kh < decltype(half_c)::value + 1; ++kh) {
            const uint32_t aa = addr_a[SLOT][kh], ab = addr_b[SLOT][kh];
            // (an array element as an asm operand inside a generic lambda does not compile: references)
            v4i &a0 = fa[kh][0], &a1 = fa[kh][1], &a2 = fa[kh][MB - 2], &a3 = fa[kh][MB - 1], &b0 = fb[kh][0], &b1 = fb[kh][1], &b2 = fb[kh][2], &b3 = fb[kh][3];
            asm volatile("ds_read_b128 %0, %1" : "=v"(a0) : "v"(aa) : "memory");
            asm volatile("ds_read_b128 %0, %1" : "=v"(b0) : "v"(ab) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(a1) : "v"(aa) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(b1) : "v"(ab) : "memory");
            if constexpr (MB == 4) asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(a2) : "v"(aa) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(b2) : "v"(ab) : "memory");
            if constexpr (MB == 4) asm volatile("ds_read_b128 %0, %1 offset:6144" : "=v"(a3) : "v"(aa) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:6144" : "=v"(b3) : "v"(ab) : "memory");
        }
    };
    auto read_stage = [&](auto slot_c) {
        read_half(slot_c, std::integral_constant<int, 0>{});
        read_half(slot_c, std::integral_constant<int, 1>{});
    };
#ifndef TPQ_STAGGER_INTERLEAVE
#define TPQ_STAGGER_INTERLEAVE 1
#endif
    // memory phase of a wavefront that also requests: TPQ_STAGGER_INTERLEAVE 0: the reads, then the requests; 1: a third
    // of the requests ahead of each half of the reads and behind them, so that the memory path has work from the start
    auto read_and_request = [&](auto read_slot, auto fill_slot, int kt_new) {
        if constexpr (TPQ_STAGGER_INTERLEAVE == 0) {
            read_stage(read_slot);
            request_stage(fill_slot, kt_new);
        } else {
            constexpr int kFirst = (kLoads + 2) / 3, kSecond = (kLoads - kFirst + 1) / 2, kThird = kLoads - kFirst - kSecond;  // 2 2 2 (2 1 1)
            request(std::integral_constant<int, 0>{}, std::integral_constant<int, kFirst>{}, fill_slot, kt_new);
            read_half(read_slot, std::integral_constant<int, 0>{});
            request(std::integral_constant<int, kFirst>{}, std::integral_constant<int, kSecond>{}, fill_slot, kt_new);
            read_half(read_slot, std::integral_constant<int, 1>{});
            request(std::integral_constant<int, kFirst + kSecond>{}, std::integral_constant<int, kThird>{}, fill_slot, kt_new);
        }
    };
    auto stage_ready = [&]() {  // every fragment read has delivered; the MFMAs that use them stay behind this point
        // (every register must appear once: a register named twice would be copied in front of the wait)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fb[0][0]), "+v"(fb[0][1]), "+v"(fb[0][2]), "+v"(fb[0][3]));
        asm volatile("" : "+v"(fa[1][0]), "+v"(fa[1][1]), "+v"(fb[1][0]), "+v"(fb[1][1]), "+v"(fb[1][2]), "+v"(fb[1][3]));
        if constexpr (MB == 4) asm volatile("" : "+v"(fa[0][MB - 2]), "+v"(fa[0][MB - 1]), "+v"(fa[1][MB - 2]), "+v"(fa[1][MB - 1]));
    };

    acc_t acc[MB][4];  // [block of 16 rows][block of 16 columns]
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = acc_t{0, 0, 0, 0};
    // W fragment first: a lane ends up with 4 consecutive n for one m.  Column blocks in snake order, so that one operand
    // changes from one instruction to the next.
    auto multiply_stage = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(kPhasePrio);
#pragma unroll
        for (int kh = 0; kh < 2; ++kh)
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const int j = (i & 1) ? 3 - jj : jj;
                    acc[i][j] = Arith::mfma(fb[kh][j], fa[kh][i], acc[i][j]);
                }
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
    };

#ifdef TPQ_STAGGER_PHASE_STAMPS
    // clock stamps of every barrier (arrival, departure), kept in s[96:99] until the following barrier, parked in LDS
    // behind the scales with a bare instruction, copied out at the end
    uint4* phase_lds = reinterpret_cast<uint4*>(lds_bytes + kRingBytes + (2 * BN + BM) * sizeof(float)) + wave * 64;
    int phase_index = 0;
    auto phase_end = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        if (phase_index > 0) {
            uint32_t t0, t1, t2, t3;
            asm volatile("s_waitcnt lgkmcnt(0)\n\tv_mov_b32 %0, s96\n\tv_mov_b32 %1, s97\n\tv_mov_b32 %2, s98\n\tv_mov_b32 %3, s99"
                         : "=v"(t0), "=v"(t1), "=v"(t2), "=v"(t3)::"s96", "s97", "s98", "s99");
            if (lane == 0 && phase_index <= 64) {
                const v4i t = {static_cast<int>(t0), static_cast<int>(t1), static_cast<int>(t2), static_cast<int>(t3)};
                const uint32_t where = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_ptr)(phase_lds + (phase_index - 1))));
                asm volatile("ds_write_b128 %0, %1" ::"v"(where), "v"(t) : "memory");
            }
        }
        ++phase_index;
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_memtime s[96:97]\n\ts_barrier\n\ts_memtime s[98:99]" ::: "memory", "s96", "s97", "s98", "s99");
        __builtin_amdgcn_sched_barrier(0);
    };
#else
    auto phase_end = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
#endif
    auto wait_loads = [&](auto allowed) { __builtin_amdgcn_s_waitcnt(vmcnt_imm(decltype(allowed)::value)); };
    // at most `stages` (0 .. S - 1, wave-uniform) whole stages of this wavefront's requests may still be outstanding
    auto wait_stages = [&](int stages) {
        bool done = false;
        static_for<0, S>([&](auto i) {
            constexpr int N = S - 1 - decltype(i)::value;  // S - 1 down to 0
            if (!done && stages >= N) {
                wait_loads(std::integral_constant<int, N * kLoads>{});
                done = true;
            }
        });
    };
    constexpr std::integral_constant<int, (S - 2) * kLoads> kSteadyWait{};  // own share of the next stage landed, the S - 2 after it may be in flight

    // ---- prologue: scales, the first stages requested, stage 0 landed ------------------------------------------------
    // The scales of the tile go to LDS by direct loads as well (64 floats per wave-level load, source index clamped at the
    // edges), ahead of the stages in every requesting wavefront's order, so the wait for stage 0 covers them; nothing
    // here is a load the compiler counts, so it inserts no wait of its own in front of the first barrier.
    if (Tile::kScaled) {
        // pieces of 64 floats: column scales 0..1, bias 2..3, row scales 4..7 (4..5); one per wavefront
        constexpr int kPieces = 8 / kRequesters;
#pragma unroll
        for (int e = 0; e < kPieces; ++e) {
            const int piece = rq * kPieces + e;
            const float* src = piece < 2 ? tile.cs : piece < 4 ? tile.bias : tile.rs;
            const int first = piece < 2 ? n0 + piece * 64 : piece < 4 ? n0 + (piece - 2) * 64 : m0 + (piece - 4) * 64;
            const int limit = piece < 4 ? N : M;
            const int idx = first + lane < limit ? first + lane : limit - 1;
            const uint32_t off = static_cast<uint32_t>(idx) * 4;
            const uint32_t dst = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_ptr)cs_lds)) + piece * 256;
            if (src != nullptr && piece < 4 + BM / 64) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(dst), "v"(off), "s"(src) : "memory", "m0");
        }
    }
    // Stages 0 .. S - 2 by everybody, stage S - 1 by group 0 only: group 1 leaves its share of it to its first memory
    // phase (phase 0, as the ring protocol has it for every later stage), which is that many loads fewer in front of the
    // first barrier; every wavefront reaches it only after the memory path has accepted all its requests.
    {
        const int mine = wave < 4 ? (nk < S ? nk : S) : (nk < S - 1 ? nk : S - 1);  // stages this wavefront requests here
        static_for<0, S>([&](auto st) {
            if (decltype(st)::value < mine) request_stage(st, decltype(st)::value);
        });
        wait_stages(mine - 1);  // stage 0 (and the scales in front of it) landed
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    TPQ_STAGGER_STAMP(1);

    // one phase pair of a wavefront; SLOT = slot of stage kt.  STEADY: every stage named exists, no conditions.
    // group 0: multiply kt | read kt + 1, request kt + S into SLOT
    auto group0_step = [&](auto slot_c, auto steady, int kt) {
        constexpr int SLOT = decltype(slot_c)::value, NEXT = (SLOT + 1) % S;
        constexpr bool STEADY = decltype(steady)::value;
        multiply_stage();
        if (STEADY) wait_loads(kSteadyWait);  // own share of kt + 1 landed (kt + 2 .. may be in flight)
        else wait_stages(nk - kt - 2 < 0 ? 0 : nk - kt - 2 < S - 2 ? nk - kt - 2 : S - 2);
        phase_end();
        if (STEADY || kt + 1 < nk) {
            if (STEADY || kt + S < nk) read_and_request(std::integral_constant<int, NEXT>{}, slot_c, kt + S);
            else read_stage(std::integral_constant<int, NEXT>{});
            stage_ready();
            phase_end();
        }
    };
    // group 1: read kt, request kt + S - 1 into the slot of kt - 1 | multiply kt
    auto group1_step = [&](auto slot_c, auto steady, int kt) {
        constexpr int SLOT = decltype(slot_c)::value, PREV = (SLOT + S - 1) % S;
        constexpr bool STEADY = decltype(steady)::value;
        if (STEADY || kt + S - 1 < nk) read_and_request(slot_c, std::integral_constant<int, PREV>{}, kt + S - 1);
        else read_stage(slot_c);
        stage_ready();
        if (STEADY) wait_loads(kSteadyWait);  // own share of kt + 1 landed (kt + 2 .. may be in flight)
        else wait_stages(nk - kt - 2 < 0 ? 0 : nk - kt - 2 < S - 2 ? nk - kt - 2 : S - 2);
        phase_end();
        multiply_stage();
        if (STEADY || kt + 1 < nk) phase_end();
    };
    constexpr std::true_type kSteady{};
    constexpr std::false_type kChecked{};

    // The steady loops are unrolled S times so that the ring slot is a constant; what is left behind them (at most
    // 2 S - 1 stages) is nested straight-line code with the conditions of the ends (a loop with a runtime slot made
    // the compiler copy the accumulators between its arms).
    int kt = 0;
    if (wave < 4) {
        read_stage(c0);
        stage_ready();
        for (; kt + 2 * S - 1 < nk; kt += S)
            static_for<0, S>([&](auto i) { group0_step(i, kSteady, kt + decltype(i)::value); });
        nested_while_below<0, 2 * S - 1>(kt, nk, [&](auto d) {  // the first of them in slot 0
            group0_step(std::integral_constant<int, decltype(d)::value % S>{}, kChecked, kt + decltype(d)::value);
        });
    } else {
        group1_step(c0, kChecked, 0);
        for (kt = 1; kt + 2 * S - 2 < nk; kt += S)
            static_for<0, S>([&](auto i) { group1_step(std::integral_constant<int, (1 + decltype(i)::value) % S>{}, kSteady, kt + decltype(i)::value); });
        nested_while_below<0, 2 * S - 2>(kt, nk, [&](auto d) {  // the first of them in slot 1
            group1_step(std::integral_constant<int, (1 + decltype(d)::value) % S>{}, kChecked, kt + decltype(d)::value);
        });
    }

    // ---- epilogue: every wavefront finishes its own 64 x 64 block ------------------------------------------------
    // Behind the last barrier nobody reads the ring and every direct load has landed, so each wavefront turns its
    // block into row order in 12 KB of its own there and stores it itself, 16 bytes per lane, whole 128-byte lines.
    // 16-bit outputs: all 64 rows at once; 32-bit outputs: two passes of 32 rows through the same 12 KB.
    TPQ_STAGGER_STAMP(2);
#ifdef TPQ_STAGGER_PHASE_STAMPS
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (blockIdx.x == 9) {
        const uint4 v = reinterpret_cast<const uint4*>(lds_bytes + kRingBytes + (2 * BN + BM) * sizeof(float))[wave * 64 + lane];
        g_stagger_stamps[(wave * 64 + lane) * 2] = (static_cast<unsigned long long>(v.y) << 32) | v.x;
        g_stagger_stamps[(wave * 64 + lane) * 2 + 1] = (static_cast<unsigned long long>(v.w) << 32) | v.z;
    }
#endif
    const bool has_bias = tile.bias != nullptr;
    constexpr int kElem = sizeof(out_t);
    constexpr int kPassBlocks = kElem == 2 ? MB : 2;             // 16-row blocks per pass
    constexpr int kWavePitch = WN * kElem + 16;                  // bytes per row of the wavefront's image
    constexpr int kRowChunks = WN * kElem / 16;                  // 16-byte chunks per row: 8 or 16
    constexpr int kRowsPerStore = kWave / kRowChunks;            // rows per wavefront store: 8 or 4
    static_assert(8 * 12288 <= kRingBytes && kPassBlocks * 16 * kWavePitch <= 12288, "eight wavefront images in the ring");
    char* img = lds_bytes + wave * 12288;
#pragma unroll
    for (int first = 0; first < MB; first += kPassBlocks) {
        float rs_r[kPassBlocks];
#pragma unroll
        for (int i = 0; i < kPassBlocks; ++i) rs_r[i] = Tile::kScaled ? rs_lds[wm * WM + (first + i) * 16 + frag_row] : 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n_wave = j * 16 + 4 * frag_chunk;  // 4 consecutive columns of the wavefront's 64
            float c4[4] = {0, 0, 0, 0}, b4[4] = {0, 0, 0, 0};
            if (Tile::kScaled) {
                const float4 c = *reinterpret_cast<const float4*>(cs_lds + wn * WN + n_wave);
                const float4 b = *reinterpret_cast<const float4*>(cs_lds + BN + wn * WN + n_wave);
                c4[0] = c.x; c4[1] = c.y; c4[2] = c.z; c4[3] = c.w;
                b4[0] = b.x; b4[1] = b.y; b4[2] = b.z; b4[3] = b.w;
            }
#pragma unroll
            for (int i = 0; i < kPassBlocks; ++i) {
                char* dst = img + (i * 16 + frag_row) * kWavePitch + n_wave * kElem;
                if constexpr (kElem == 2) {
                    float f[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) f[t] = Tile::value(acc[first + i][j][t], rs_r[i], c4[t], b4[t], has_bias);
                    *reinterpret_cast<uint2*>(dst) = make_uint2(Tile::pack2(f[0], f[1]), Tile::pack2(f[2], f[3]));
                } else {
                    out_t vals[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) vals[t] = Tile::convert(acc[first + i][j][t], rs_r[i], c4[t], b4[t], has_bias);
                    *reinterpret_cast<uint4*>(dst) = make_uint4(__builtin_bit_cast(uint32_t, vals[0]), __builtin_bit_cast(uint32_t, vals[1]),
                                                                __builtin_bit_cast(uint32_t, vals[2]), __builtin_bit_cast(uint32_t, vals[3]));
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wavefront's own LDS writes, in order with its reads
#pragma unroll
        for (int it = 0; it < kPassBlocks * 16 / kRowsPerStore; ++it) {
            const int row = it * kRowsPerStore + lane / kRowChunks, col = (lane % kRowChunks) * (16 / kElem);
            const int m = m0 + wm * WM + first * 16 + row, n = n0 + wn * WN + col;
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
    TPQ_STAGGER_STAMP(3);
}

// row_bytes = K * sizeof(element): a multiple of 128 below 2^23
template <class Arith, int MB, class Tile>
int launch_stagger_bytes(const void* a, const void* w, int64_t M, int64_t N, int64_t row_bytes, Tile tile, hipStream_t s, int slices, const char* what) {
    constexpr int BM = 64 * MB;
    constexpr size_t smem = static_cast<size_t>(kDmaStages) * (BM + 128) * kDmaRowBytes + (2 * 128 + BM) * sizeof(float) + kStaggerStampBytes;
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + 127) / 128);
    TPQ_REQUIRE(tiles <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "staggered gemm: too many tiles");
    TPQ_REQUIRE(row_bytes % kDmaRowBytes == 0 && row_bytes < (1 << 23), TPQ_ERR_INVALID_VALUE, "staggered gemm: a row of k must be a multiple of 128 bytes below 2^23");
    auto kernel = gemm_stagger_kernel<Tile, Arith, MB>;
    static std::atomic<uint64_t> configured{0};  // per instantiation
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), smem, configured, what)) return rc;
    const int vector_stores = (N * sizeof(typename Tile::out_t)) % 16 == 0 && aligned(tile.out, 16);
    kernel<<<dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(slices)), 512, smem, s>>>(
        static_cast<const char*>(a), static_cast<const char*>(w), static_cast<int>(M), static_cast<int>(N), static_cast<int>(row_bytes), tile, vector_stores, slices);
    return check_launch(what);
}

template <class Tile>
int launch_stagger(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Tile tile, hipStream_t s, int slices = 1) {
    return launch_stagger_bytes<ArithI8, 4>(a, w, M, N, K, tile, s, slices, "int8 mfma gemm (staggered)");
}

}  // namespace
}  // namespace tpq
