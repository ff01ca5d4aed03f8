// Ternary-weight product for 33 rows and more (BitNet prefill chunks), K % 128 == 0: every load of a workgroup
// requested before the first one is used.
//
// The work is small (128 x 6912 x 2560 is 4.5 GOP, a microsecond of matrix-core time; the packed weight is
// 4.4 MB), so what decides the time is the chain of dependent steps in a workgroup and how often the activations
// cross the vector path.  A workgroup of 16 wavefronts owns a tile of 32 rows x 128 channels over a range of
// U <= 20 units of 128 k:
//
//   * all 1024 threads request their share of the 32 x 128 U bytes of activations (16-byte chunks, a wavefront
//     load = 1 KB contiguous) and their own packed weights up front, straight-line; nothing is waited for until
//     everything has been asked for.  The epilogue's row scales and bias are asked for first and parked in LDS;
//   * the activations go through LDS once: each 16-byte chunk is transposed as a 4 x 4 byte matrix on its way
//     (the cheap expansion of a packed dword yields the codes of one field position of its four bytes, so the
//     k order of the MFMA operands is field-major; see ternary_decode_mfma.h), a 64-byte segment becomes four
//     16-byte MFMA operands (operand f = field f of its four chunks), kept in slot (8 unit + 4 half + f) ^ (row % 16)
//     of the row (rows are a multiple of 256 bytes apart): the 16 lanes that a 16-byte LDS read serves together
//     hit 16 different bank groups;
//   * the packed weights are fetched in whole 128-byte lines (a load costs the vector memory path the lines it
//     touches) and reach MFMA order through small LDS areas of their own;
//   * one barrier, then wavefront (nb, kp) multiplies channel block nb with its units (slab_unit_of):
//     v_mfma_i32_32x32x32_i8, A = activations from LDS, B = weight fields moved to the top of their bytes in
//     registers, four MFMAs per unit;
//   * the four k-parts meet in LDS (the slab's space, after a second barrier); every thread finishes and stores
//     four consecutive columns of one row.
//
// Where the time goes (clock stamps at 128 x 6912 x 2560, 216 workgroups, 13,200 clocks): the requests of a workgroup
// are accepted at about 2.7 clocks per cache line they touch (the last wavefront has its requests out after 3,700
// clocks; 6,300 with the weights as 64-byte runs of 16 rows, which made the kernel 14,900 clocks), and the last
// wavefront's activations are in LDS after 6,100; from then
// on 16 wavefronts on four SIMDs pay four clocks of a SIMD per vector instruction and wavefront, so a hundred
// instructions per wavefront are 1600 clocks: the expansion of the weights, the sums and the epilogue are
// instruction issue, not memory (without the weight loads the phases behind the barrier take as long as with them).
//
// With more than one split of K the exact int32 sums of split z go to partial[z][M][N] and ternary_slab_finish_kernel
// adds them and applies the epilogue; with one split the epilogue is applied here.
#pragma once

#include "ternary_decode_mfma.h"

namespace tpq {
namespace {

constexpr int kSlabRows = 32, kSlabChannels = 128, kSlabThreads = 1024;
constexpr int kSlabUnitsPerWave = 5, kSlabKParts = 4, kSlabUnits = kSlabUnitsPerWave * kSlabKParts;  // 20 units = 2560 k
constexpr int kSlabChunkRounds = kSlabRows * kSlabUnits * 8 / kSlabThreads;                          // 5 chunks of 16 bytes per thread
constexpr int kSlabXchPitch = 144;                                                                   // bytes between the rows of the weight exchange areas in LDS
constexpr int kSlabXchBytes = (4 * 32 + 16 * 16) * kSlabXchPitch;                                    // units 16 .. 19 of four channel blocks + 16 rows per wavefront

// x: [M][K] int8; packed: [N][K/4]; units_per_split units of 128 k per workgroup (<= kSlabUnits), split z takes the
// units z units_per_split ...; lds_main_bytes: size of the slab / k-part area; 32 row scales and 128 bias values sit behind it;
// grid: 8 m_tiles ceil(n_tiles splits / 8) workgroups (see the id mapping below); partial: [gridDim.z][M][N] int32 or null (one split: the epilogue stores)
#ifdef TPQ_SLAB_STAMPS
__device__ unsigned long long g_slab_stamps[16 * 16];
#define TPQ_STAMP(I) do { if (blockIdx.x == 8 && lane == 0) g_slab_stamps[(I) * 16 + wave] = __builtin_amdgcn_s_memtime(); } while (0)
#else
#define TPQ_STAMP(I) do { } while (0)
#endif

// Unit j of k-part kp.  A row of packed weights holds four units per 128-byte cache line: the four units of a line go to
// one wavefront, which fetches the line whole (dealt round-robin, unit kp + 4 j, every line was fetched by four
// wavefronts at four different times, four times the traffic between the caches).  Units 16..19 go one to each k-part.
__device__ __forceinline__ constexpr int slab_unit_of(int kp, int j) { return j < 4 ? 4 * kp + j : 16 + kp; }
static_assert(kSlabUnitsPerWave == 5 && kSlabKParts == 4, "slab_unit_of deals 20 units");

template <class Epilogue>
__global__ __launch_bounds__(kSlabThreads) void ternary_slab_kernel(const int8_t* __restrict__ x, const uint8_t* __restrict__ packed,
                                                                   int M, int N, int K, int units_per_split, int lds_main_bytes, int m_tiles, int n_tiles, int splits,
                                                                   int32_t* __restrict__ partial, Epilogue ep) {
    extern __shared__ __align__(16) unsigned char slab_lds[];  // [32 rows][U units][8 slots of 16 bytes]; later the k-part sums
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nb = wave & 3, kp = wave >> 2;
    // The row tiles of one (channel tile, split) read the same packed weights: they get workgroup ids that are equal
    // mod 8, so they run on the same XCD and the weights are brought into one L2, not into as many as there are row
    // tiles.  id = 8 (m_tile + m_tiles * (slab / 8)) + slab % 8 with slab = n_tile + n_tiles * split; the grid is
    // padded to a multiple of 8 slabs.
    const int slab_id = (blockIdx.x & 7) + 8 * ((blockIdx.x >> 3) / m_tiles), m_tile = (blockIdx.x >> 3) % m_tiles;
    if (slab_id >= n_tiles * splits) return;  // padding (whole workgroup, before any barrier)
    const int split = slab_id / n_tiles, n_tile = slab_id - split * n_tiles;
    const int n0 = n_tile * kSlabChannels, m0 = m_tile * kSlabRows;
    const int units_total = K >> 7;
    const int unit0 = split * units_per_split;
    const int U = units_total - unit0 < units_per_split ? units_total - unit0 : units_per_split;  // this workgroup's units, >= 1

    TPQ_STAMP(0);
    // the epilogue's row scales and bias, asked for ahead of everything else and parked in LDS: fetched at the end they
    // are a trip to memory that nothing covers
    float scale_word = 0.0f;
    if (partial == nullptr) {
        if (tid < kSlabRows) scale_word = ep.row_scale_of(m0 + tid < M ? m0 + tid : M - 1);
        else if (tid < kSlabRows + kSlabChannels) scale_word = ep.bias_of(n0 + tid - kSlabRows < N ? n0 + tid - kSlabRows : N - 1);
    }
    // ---- requests ---------------------------------------------------------------------------------------------
    // activations: 16-byte chunks, 32 threads per row (thread t: row t / 32, chunks t % 32, t % 32 + 32, ...): a
    // wavefront load is two runs of 512 contiguous bytes (eight cache lines; a 64-byte segment per lane made it 64
    // lines, and the texture path's line look-ups were the time of the whole kernel)
    uint4 xa[kSlabChunkRounds];
    const int row_slots = 8 * (U + (U & 1));  // an even number of units per row: the swizzle below swaps neighbouring units
    const int x_row = tid >> 5, x_lane = tid & 31;
    {
        const int m = m0 + x_row < M ? m0 + x_row : M - 1;
        const uint4* src = reinterpret_cast<const uint4*>(x + static_cast<size_t>(m) * K + (static_cast<size_t>(unit0) << 7));
#pragma unroll
        for (int r = 0; r < kSlabChunkRounds; ++r) {
            const int cc = x_lane + 32 * r;  // chunk cc of the row: unit cc / 8, half (cc / 4) % 2, c = cc % 4
            xa[r] = src[cc < 8 * U ? cc : 0];
        }
    }
    // weights of wavefront (nb, kp).  The MFMA wants lane (n, half) to hold the 16 bytes (64 codes) of half `half` of
    // a unit for row n0 + 32 nb + n: asked for like that, a wavefront load takes 32 bytes out of 32 cache lines, and what
    // a load costs the vector memory path is the lines it touches (about 2.7 clocks each: the requests of the last
    // wavefront were accepted 6,300 clocks into the kernel when the weights came as 64-byte runs of 16 rows and the fifth
    // unit in MFMA order, 16 and 32 lines per load).  So the weights are fetched in whole lines: the four units of the
    // wavefront's own line (4 kp .. 4 kp + 3 are the 128 bytes of one line of a row) as four loads of eight rows x 128
    // bytes, lane l = row l / 8 of the eight, 16-byte chunk l % 8 (unit 4 kp + chunk / 2, half chunk % 2); and of the
    // line that holds the units 16 .. 19 the wavefront fetches rows 8 kp .. 8 kp + 7 of its channel block for all four
    // k-parts.  Both go through LDS on their way into MFMA order (below).
    const int wn = lane & 31, half = lane >> 5;
    const int w_row8 = lane >> 3, w_chunk = lane & 7;
    uint4 wl[4], wl5;
    {
        const size_t pitch = static_cast<size_t>(K >> 2);
        const unsigned char* const base = packed + (static_cast<size_t>(unit0) << 5);
        const int u_own = 4 * kp + (w_chunk >> 1), u_fifth = 16 + (w_chunk >> 1);
        // a unit past the end of the split re-reads the first bytes of the row's range and is not multiplied
        const int off_own = u_own < U ? u_own * 32 + (w_chunk & 1) * 16 : 0;
        const int off_fifth = u_fifth < U ? u_fifth * 32 + (w_chunk & 1) * 16 : 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = n0 + 32 * nb + 8 * i + w_row8;
            wl[i] = nt_load(reinterpret_cast<const uint4*>(base + (row < N ? row : N - 1) * pitch + off_own));
        }
        const int row = n0 + 32 * nb + 8 * kp + w_row8;
        wl5 = nt_load(reinterpret_cast<const uint4*>(base + (row < N ? row : N - 1) * pitch + off_fifth));
    }

    TPQ_STAMP(1);
    // ---- activations into LDS, in MFMA operand order ------------------------------------------------------
    // chunk c of a segment, transposed, is dword c of each of the segment's four operands: operand f of segment
    // (unit, half) sits in slot (8 unit + 4 half + f) ^ (row % 16) of the row.
    float* const scale_lds = reinterpret_cast<float*>(slab_lds + lds_main_bytes);  // [32] row scales, [128] bias (one split only)
    if (partial == nullptr && tid < kSlabRows + kSlabChannels) scale_lds[tid] = scale_word;
#pragma unroll
    for (int r = 0; r < kSlabChunkRounds; ++r) {
        const int cc = x_lane + 32 * r;
        if (cc < 8 * U) {
            const v4i t = transpose_4x4_bytes(xa[r]);
            const int dst = (x_row * row_slots + ((cc & ~3) ^ (x_row & 15))) * 16 + (cc & 3) * 4;
#pragma unroll
            for (int f = 0; f < 4; ++f)  // f is xor-ed into the swizzled slot: row_slots is a multiple of 16
                *reinterpret_cast<int*>(slab_lds + (dst ^ (f * 16))) = t[f];
        }
    }
    // ---- weights into MFMA order through LDS ------------------------------------------------------------------
    // Rows 144 bytes apart: the 16 lanes a 16-byte read serves together (rows n .. n + 15, one chunk) hit 16 different
    // bank groups.  The own line: a wavefront-private area of 16 rows, used twice (rows 0 .. 15, then 16 .. 31 of the
    // channel block; LDS accesses of one wavefront execute in order, no barrier).  The line of the units 16 .. 19: an area
    // per channel block that the four k-parts fill together, read behind the barrier that the activations need anyway.
    uint4 wq[kSlabUnitsPerWave];  // [j]: unit slab_unit_of(kp, j) in MFMA order
    {
        unsigned char* const xch = slab_lds + lds_main_bytes + (kSlabRows + kSlabChannels) * sizeof(float);
        unsigned char* const fifth = xch + (nb * 32) * kSlabXchPitch;
        *reinterpret_cast<uint4*>(fifth + (8 * kp + w_row8) * kSlabXchPitch + w_chunk * 16) = wl5;
        unsigned char* const mine = xch + 4 * 32 * kSlabXchPitch + wave * 16 * kSlabXchPitch;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            *reinterpret_cast<uint4*>(mine + w_row8 * kSlabXchPitch + w_chunk * 16) = wl[2 * h];
            *reinterpret_cast<uint4*>(mine + (8 + w_row8) * kSlabXchPitch + w_chunk * 16) = wl[2 * h + 1];
            __builtin_amdgcn_wave_barrier();
            if ((wn >> 4) == h) {
#pragma unroll
                for (int j = 0; j < 4; ++j) wq[j] = *reinterpret_cast<const uint4*>(mine + (wn & 15) * kSlabXchPitch + (2 * j + half) * 16);
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
    TPQ_STAMP(2);
    __syncthreads();
    TPQ_STAMP(3);
    wq[4] = *reinterpret_cast<const uint4*>(slab_lds + lds_main_bytes + (kSlabRows + kSlabChannels) * sizeof(float) +
                                            (nb * 32 + wn) * kSlabXchPitch + (2 * kp + half) * 16);

    // ---- wavefront (nb, kp): 32 rows x 32 channels over its units ------------------------------------------
    // A 2-bit field at the top of a byte is the code times 64 as a signed byte (0b11 -> -64, 0b10 -> -128: the
    // reference's sign extension of the field, tensorplay/ao/quantization/bitnet.py:75-79), so field f of the four
    // bytes of a word is (w << 2 f) & 0xC0C0C0C0: seven instructions per 16 codes, every field at the same weight, no
    // offset to take out afterwards.  |sum| <= 2560 * 127 * 128 < 2^31.  Two accumulators, so that consecutive MFMAs
    // do not wait for each other; the factor 64 is taken out of the finished sum with an exact shift.
    v16i acc0, acc1;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0;
    // A: lane (m, half) reads row m; operand f of unit u: slot (8 u + 4 half + f) ^ (m % 16) = 8 (u ^ (m / 8 % 2)) + ((4 half + f) ^ (m % 8))
    const unsigned char* a_row = slab_lds + static_cast<size_t>(wn) * row_slots * 16;
    int a_off[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) a_off[f] = ((4 * half + f) ^ (wn & 7)) * 16;
#pragma unroll
    for (int j = 0; j < kSlabUnitsPerWave; ++j) {
        const int u = slab_unit_of(kp, j);
        if (u < U) {  // wave-uniform
            const uint32_t w0 = wq[j].x, w1 = wq[j].y, w2 = wq[j].z, w3 = wq[j].w;
            const unsigned char* a_unit = a_row + (u ^ ((wn >> 3) & 1)) * 128;  // neighbouring units swapped for rows 8..15, 24..31
            constexpr uint32_t kTop = 0xC0C0C0C0u;
            {
                const v4i fb = {static_cast<int>(w0 & kTop), static_cast<int>(w1 & kTop), static_cast<int>(w2 & kTop), static_cast<int>(w3 & kTop)};
                acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i*>(a_unit + a_off[0]), fb, acc0, 0, 0, 0);
            }
            {
                const v4i fb = {static_cast<int>((w0 << 2) & kTop), static_cast<int>((w1 << 2) & kTop), static_cast<int>((w2 << 2) & kTop),
                                static_cast<int>((w3 << 2) & kTop)};
                acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i*>(a_unit + a_off[1]), fb, acc1, 0, 0, 0);
            }
            {
                const v4i fb = {static_cast<int>((w0 << 4) & kTop), static_cast<int>((w1 << 4) & kTop), static_cast<int>((w2 << 4) & kTop),
                                static_cast<int>((w3 << 4) & kTop)};
                acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i*>(a_unit + a_off[2]), fb, acc0, 0, 0, 0);
            }
            {
                const v4i fb = {static_cast<int>((w0 << 6) & kTop), static_cast<int>((w1 << 6) & kTop), static_cast<int>((w2 << 6) & kTop),
                                static_cast<int>((w3 << 6) & kTop)};
                acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i*>(a_unit + a_off[3]), fb, acc1, 0, 0, 0);
            }
        }
    }
    v16i acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = acc0[v] + acc1[v];  // 64 times the sum

    // ---- add the k-parts: every wavefront parks its sums in LDS and finishes a quarter of its block -------------
    TPQ_STAMP(4);
    __syncthreads();
    TPQ_STAMP(5);
    int* const part = reinterpret_cast<int*>(slab_lds);  // [4 kp][4 nb][16][64]: 64 KB
#pragma unroll
    for (int v = 0; v < 16; ++v) part[((kp * 4 + nb) * 16 + v) * kWave + lane] = acc[v];
    __syncthreads();
    TPQ_STAMP(6);
    {
        // C fragment of a 32 x 32 block: register v of lane l is row 8 (v / 4) + 4 (l / 32) + v % 4, column l % 32.
        // Thread -> (block, register v, lanes 4 c .. 4 c + 3): four consecutive columns of one row, one 16-byte read per
        // k-part and one vector store
        const int c = tid & 15, v = (tid >> 4) & 15, block = tid >> 8;
        int sum[4] = {0, 0, 0, 0};
#pragma unroll
        for (int p = 0; p < kSlabKParts; ++p) {
            const int4 q = *reinterpret_cast<const int4*>(part + ((p * 4 + block) * 16 + v) * kWave + 4 * c);
            sum[0] += q.x; sum[1] += q.y; sum[2] += q.z; sum[3] += q.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) sum[e] >>= 6;  // exact: every term is a multiple of 64
        const int row = 8 * (v >> 2) + 4 * (c >> 3) + (v & 3), col = 32 * block + ((4 * c) & 31);
        const int m = m0 + row, n = n0 + col;
        if (m < M && n < N) {
            const int count = N - n < 4 ? N - n : 4;
            const int64_t idx = static_cast<int64_t>(m) * N + n;
            if (partial) {
                int32_t* const mine = partial + static_cast<size_t>(split) * M * N;  // 16-byte aligned (launcher)
                if (count == 4 && (N & 3) == 0 && ((static_cast<size_t>(split) * M * N) & 3) == 0) {
                    *reinterpret_cast<int4*>(mine + idx) = make_int4(sum[0], sum[1], sum[2], sum[3]);
                } else {
                    for (int e = 0; e < count; ++e) mine[idx + e] = sum[e];
                }
            } else {
                const float4 b = *reinterpret_cast<const float4*>(scale_lds + kSlabRows + col);  // fetched at the start of the kernel
                const float bias_n[4] = {b.x, b.y, b.z, b.w};
                ep.store_scaled_run(idx, sum, scale_lds[row], bias_n, count, count == 4 && (N & 3) == 0 && ep.runs_aligned());
            }
        }
    }
    TPQ_STAMP(7);
}

// out = epilogue(sum over the splits): a thread takes four consecutive columns of one row (grid.y = row, so no
// division per element; 16-byte loads of the partial sums, one vector store where the row pitch allows)
template <class Epilogue>
__global__ __launch_bounds__(256) void ternary_slab_finish_kernel(const int32_t* __restrict__ partial, int splits, int M, int N, Epilogue ep) {
    const int m = blockIdx.y;
    const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (n >= N) return;
    const int count = N - n < 4 ? N - n : 4;
    const int64_t total = static_cast<int64_t>(M) * N, idx = static_cast<int64_t>(m) * N + n;
    const bool whole = count == 4 && (N & 3) == 0;  // the partial matrices are 16-byte aligned (launcher) and M N is a multiple of 4
    const float row_scale = ep.row_scale_of(m);
    float bias_n[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) bias_n[e] = ep.bias_of(e < count ? n + e : n);
    int v[4] = {0, 0, 0, 0};
    if (whole) {
        // four splits requested together (a loop of load and add would wait for memory once per split); a batch past
        // the last split asks for the last one again and leaves it out of the sum
        for (int s0 = 0; s0 < splits; s0 += 4) {
            int4 q[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) q[j] = *reinterpret_cast<const int4*>(partial + (s0 + j < splits ? s0 + j : splits - 1) * total + idx);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (s0 + j < splits) { v[0] += q[j].x; v[1] += q[j].y; v[2] += q[j].z; v[3] += q[j].w; }
        }
    } else {
        for (int s = 0; s < splits; ++s)
            for (int e = 0; e < count; ++e) v[e] += partial[s * total + idx + e];
    }
    ep.store_scaled_run(idx, v, row_scale, bias_n, count, whole && ep.runs_aligned());
}

// Splits of K for the slab kernel (1: no workspace needed); 0 when the kernel does not take the shape.
// It is built for one pass of workgroups over the chip: every 32 rows expand the packed weights again, which the
// tile kernel of ternary_gemm_kernel.h does once per 128 (or 64) rows.  Measured (us, bf16 out, slab / tile kernel):
//   2560 -> 6912: 7.1 / 9.6 at 64 rows, 7.4 / 11.3 at 128, 17.0 / 15.9 at 256 (two passes of workgroups)
//   6912 -> 2560 (three splits): 9.5 / 16.2 at 64, 10.8 / 16.8 at 128
//   two splits: 4096 -> 4096 9.5 / 11.4 at 33 rows, 9.9 / 11.7 at 64, 11.4 / 11.8 at 128; 5120 -> 4096 11.6 / 13.5 at
//   128; 4096 -> 2048 9.9 / 11.7 at 128; 3072 -> 4096 9.6 / 10.0 at 65 but 10.9 / 10.2 at 128: with two splits the second
//   kernel that adds them costs what the shorter chain saves when the splits are short, so above 64 rows two
//   splits are taken from K = 4096 on
// Letting the splits meet inside the kernel (every workgroup leaves its sums with agent-scope stores and counts itself
// in, the last one adds and finishes) was built and is slower than the second launch at three splits (6912 -> 2560:
// 13.4 against 12.7 us at 128 rows, 11.6 against 10.1 at 33, with the kernel as it was then): store acknowledgement,
// counter and the reads of the other sums are three trips to memory in a row, a launch and one trip are less.
inline int ternary_slab_splits(int64_t M, int64_t N, int64_t K, int compute_units = 256) {
    if (M < 33 || K % 128 != 0 || K < 128 || M > 0x7FFFFFFF / 2 || N > 0x7FFFFFFF / 2 || K > 0x7FFFFFFF / 2) return 0;
    const int64_t units = K / 128;
    const int64_t splits = (units + kSlabUnits - 1) / kSlabUnits;
    const int64_t workgroups = ((M + kSlabRows - 1) / kSlabRows) * ((N + kSlabChannels - 1) / kSlabChannels) * splits;
    if (workgroups > compute_units || (splits == 2 && M > 64 && units < 32) || splits > 8) return 0;
    return static_cast<int>(splits);
}

template <class Epilogue>
int launch_ternary_slab(const int8_t* x, const uint8_t* packed, int64_t M, int64_t N, int64_t K, int splits, int32_t* partial,
                        Epilogue ep, hipStream_t s) {
    const int units = static_cast<int>(K / 128);
    const int per_split = (units + splits - 1) / splits;
    const size_t slab_bytes = static_cast<size_t>(kSlabRows) * (per_split + (per_split & 1)) * 128;
    const size_t part_bytes = static_cast<size_t>(16) * 16 * kWave * sizeof(int);  // 64 KB
    const size_t main_bytes = slab_bytes > part_bytes ? slab_bytes : part_bytes;
    const size_t smem = main_bytes + (kSlabRows + kSlabChannels) * sizeof(float) + kSlabXchBytes;
    auto kernel = ternary_slab_kernel<Epilogue>;
    static std::atomic<uint64_t> configured{0};  // per instantiation
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), static_cast<size_t>(kSlabRows) * kSlabUnits * 128 + (kSlabRows + kSlabChannels) * sizeof(float) + kSlabXchBytes, configured, "ternary slab")) return rc;
    const int64_t n_tiles = (N + kSlabChannels - 1) / kSlabChannels, m_tiles = (M + kSlabRows - 1) / kSlabRows;
    const int64_t gx = 8 * m_tiles * ((n_tiles * splits + 7) / 8);
    TPQ_REQUIRE(gx <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "ternary slab: shape too large");
    kernel<<<dim3(static_cast<unsigned>(gx)), kSlabThreads, smem, s>>>(
        x, packed, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), per_split, static_cast<int>(main_bytes),
        static_cast<int>(m_tiles), static_cast<int>(n_tiles), splits, splits > 1 ? partial : nullptr, ep);
    if (int rc = check_launch("tpq_ternary_mm (slab)")) return rc;
    if (splits > 1) {
        TPQ_REQUIRE(M <= 65535, TPQ_ERR_INVALID_VALUE, "ternary slab: too many rows for the finishing launch");
        ternary_slab_finish_kernel<Epilogue><<<dim3(static_cast<unsigned>((N + 1023) / 1024), static_cast<unsigned>(M)), 256, 0, s>>>(
            partial, splits, static_cast<int>(M), static_cast<int>(N), ep);
        return check_launch("tpq_ternary_mm (slab, finish)");
    }
    return TPQ_OK;
}

}  // namespace
}  // namespace tpq
