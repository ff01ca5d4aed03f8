// Ternary-weight product for 33 rows and more (BitNet prefill chunks), K % 128 == 0: every load of a workgroup
// requested before the first one is used.
//
// The work is small (128 x 6912 x 2560 is 4.5 GOP, a microsecond of matrix-core time; the packed weight is
// 4.4 MB), so what decides the time is the chain of dependent steps in a workgroup and how often the activations
// cross the vector path.  A workgroup of 16 wavefronts owns a tile of 32 rows x 128 channels over a range of
// U <= 20 units of 128 k:
//
//   * all 1024 threads request their share of the 32 x 128 U bytes of activations (16-byte chunks, a wavefront
//     load = 1 KB contiguous) and their own packed weights (one 16-byte load = 64 codes per unit) up front,
//     straight-line; nothing is waited for until everything has been asked for;
//   * the activations go through LDS once: each 16-byte chunk is transposed as a 4 x 4 byte matrix on its way
//     (the cheap expansion of a packed dword yields the codes of one field position of its four bytes, so the
//     k order of the MFMA operands is field-major; see ternary_decode_mfma.h), a 64-byte segment becomes four
//     16-byte MFMA operands (operand f = field f of its four chunks), kept in slot (8 unit + 4 half + f) ^ (row % 16)
//     of the row (rows are a multiple of 256 bytes apart): the 16 lanes that a 16-byte LDS read serves together
//     hit 16 different bank groups;
//   * one barrier, then wavefront (nb, kp) multiplies channel block nb with the units kp, kp + 4, ... :
//     v_mfma_i32_32x32x32_i8, A = activations from LDS, B = weight fields masked out of the packed words in
//     registers (5 instructions per 16 codes: the expansion is the vector ALU's whole load in this phase, and
//     with 3 instructions per four codes it, not the matrix core, set the time), four MFMAs per unit;
//   * the four k-parts meet in LDS (the slab's space, after a second barrier); every wavefront finishes and
//     stores a quarter of its block.
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

// x: [M][K] int8; packed: [N][K/4]; units_per_split units of 128 k per workgroup (<= kSlabUnits), split z takes the
// units z units_per_split ...; lds_main_bytes: size of the slab / k-part area, the 32 row sums sit behind it;
// grid: 8 m_tiles ceil(n_tiles splits / 8) workgroups (see the id mapping below); partial: [gridDim.z][M][N] int32 or null (one split: the epilogue stores)
#ifdef TPQ_SLAB_STAMPS
__device__ unsigned long long g_slab_stamps[16 * 16];
#define TPQ_STAMP(I) do { if (blockIdx.x == 8 && lane == 0) g_slab_stamps[(I) * 16 + wave] = __builtin_amdgcn_s_memtime(); } while (0)
#else
#define TPQ_STAMP(I) do { } while (0)
#endif

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
    // weights: lane (n, half) of wavefront (nb, kp): row n0 + 32 nb + n, the 16 bytes (64 codes) of half `half` of the unit
    const int wn = lane & 31, half = lane >> 5;
    uint4 wq[kSlabUnitsPerWave];
    {
        const int n = n0 + 32 * nb + wn < N ? n0 + 32 * nb + wn : N - 1;
        const uint4* src = reinterpret_cast<const uint4*>(packed + static_cast<size_t>(n) * (K >> 2) + (static_cast<size_t>(unit0) << 5)) + half;
#pragma unroll
        for (int j = 0; j < kSlabUnitsPerWave; ++j) {
            const int u = kp + kSlabKParts * j;
            wq[j] = nt_load(src + (u < U ? u : 0) * 2);  // a unit past the end re-reads unit 0 and is not multiplied
        }
    }

    TPQ_STAMP(1);
    // ---- activations into LDS, in MFMA operand order ------------------------------------------------------
    // chunk c of a segment, transposed, is dword c of each of the segment's four operands: operand f of segment
    // (unit, half) sits in slot (8 unit + 4 half + f) ^ (row % 16) of the row.  The codes are multiplied as
    // unsigned fields with the sign bit flipped (code = (field ^ 2) - 2), so the row sums of the activations
    // are needed once per row: every thread adds its chunks, the 32 threads of a row meet through the lanes.
    int* const row_sum = reinterpret_cast<int*>(slab_lds + lds_main_bytes);  // [32]
    {
        int mine = 0;
#pragma unroll
        for (int r = 0; r < kSlabChunkRounds; ++r) {
            const int cc = x_lane + 32 * r;
            if (cc < 8 * U) {
                const v4i t = transpose_4x4_bytes(xa[r]);
                const int dst = (x_row * row_slots + ((cc & ~3) ^ (x_row & 15))) * 16 + (cc & 3) * 4;
#pragma unroll
                for (int f = 0; f < 4; ++f) {  // f is xor-ed into the swizzled slot: row_slots is a multiple of 16
                    *reinterpret_cast<int*>(slab_lds + (dst ^ (f * 16))) = t[f];
                    mine = __builtin_amdgcn_sdot4(t[f], 0x01010101, mine, false);
                }
            }
        }
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) mine += __shfl_xor(mine, off, kWave);
        if (x_lane == 0) row_sum[x_row] = mine;
    }
    TPQ_STAMP(2);
    __syncthreads();
    TPQ_STAMP(3);

    // ---- wavefront (nb, kp): 32 rows x 32 channels over its units ------------------------------------------
    // Field f of the sign-flipped word, left where it is: w & mask is the field times 16, 4, 1 (f = 1, 2, 3); the top
    // field would overflow a signed byte there and is moved down one bit first (times 32).  One accumulator per
    // field position, put together with exact shifts at the end: 5 instructions per 16 codes.
    v16i acc0, acc1, acc2, acc3;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = acc2[v] = acc3[v] = 0;
    // A: lane (m, half) reads row m; operand f of unit u: slot (8 u + 4 half + f) ^ (m % 16) = 8 (u ^ (m / 8 % 2)) + ((4 half + f) ^ (m % 8));
    // the units of a wavefront (kp, kp + 4, ...) have the parity of kp, so the swap of neighbours is one offset per lane
    const unsigned char* a_row = slab_lds + static_cast<size_t>(wn) * row_slots * 16 + ((wn & 8) ? ((kp & 1) ? -128 : 128) : 0);
    int a_off[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) a_off[f] = ((4 * half + f) ^ (wn & 7)) * 16;
#pragma unroll
    for (int j = 0; j < kSlabUnitsPerWave; ++j) {
        const int u = kp + kSlabKParts * j;
        if (u < U) {  // wave-uniform
            const uint32_t w0 = wq[j].x ^ 0xAAAAAAAAu, w1 = wq[j].y ^ 0xAAAAAAAAu, w2 = wq[j].z ^ 0xAAAAAAAAu, w3 = wq[j].w ^ 0xAAAAAAAAu;
            const unsigned char* a_unit = a_row + u * 128;
            {
                const v4i fb = {static_cast<int>((w0 >> 1) & 0x60606060u), static_cast<int>((w1 >> 1) & 0x60606060u),
                                static_cast<int>((w2 >> 1) & 0x60606060u), static_cast<int>((w3 >> 1) & 0x60606060u)};
                acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i*>(a_unit + a_off[0]), fb, acc0, 0, 0, 0);
            }
            {
                const v4i fb = {static_cast<int>(w0 & 0x30303030u), static_cast<int>(w1 & 0x30303030u), static_cast<int>(w2 & 0x30303030u),
                                static_cast<int>(w3 & 0x30303030u)};
                acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i*>(a_unit + a_off[1]), fb, acc1, 0, 0, 0);
            }
            {
                const v4i fb = {static_cast<int>(w0 & 0x0C0C0C0Cu), static_cast<int>(w1 & 0x0C0C0C0Cu), static_cast<int>(w2 & 0x0C0C0C0Cu),
                                static_cast<int>(w3 & 0x0C0C0C0Cu)};
                acc2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i*>(a_unit + a_off[2]), fb, acc2, 0, 0, 0);
            }
            {
                const v4i fb = {static_cast<int>(w0 & 0x03030303u), static_cast<int>(w1 & 0x03030303u), static_cast<int>(w2 & 0x03030303u),
                                static_cast<int>(w3 & 0x03030303u)};
                acc3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i*>(a_unit + a_off[3]), fb, acc3, 0, 0, 0);
            }
        }
    }
    v16i acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = (acc0[v] >> 5) + (acc1[v] >> 4) + (acc2[v] >> 2) + acc3[v];  // exact: multiples of 32, 16, 4

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
        // C fragment of a 32 x 32 block: lane holds column lane % 32, rows 8 (v / 4) + 4 (lane / 32) + v % 4;
        // wavefront (nb, kp) takes v = 4 kp .. 4 kp + 3: rows 8 kp + 4 (lane / 32) + 0..3
        int sum[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sum[i] = 0;
#pragma unroll
            for (int p = 0; p < kSlabKParts; ++p) sum[i] += part[((p * 4 + nb) * 16 + 4 * kp + i) * kWave + lane];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) sum[i] -= 2 * row_sum[8 * kp + 4 * half + i];
        const int n = n0 + 32 * nb + wn;
        const int m_first = m0 + 8 * kp + 4 * half;
        if (n < N) {
            if (partial) {
                int32_t* const mine = partial + static_cast<size_t>(split) * M * N;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (m_first + i < M) mine[static_cast<int64_t>(m_first + i) * N + n] = sum[i];
            } else {
                float row_scale[4];  // all of them before the first store
#pragma unroll
                for (int i = 0; i < 4; ++i) row_scale[i] = ep.row_scale_of(m_first + i < M ? m_first + i : M - 1);
                const float bias_n = ep.bias_of(n);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (m_first + i < M) ep.store_scaled(static_cast<int64_t>(m_first + i) * N + n, sum[i], row_scale[i], bias_n);
            }
        }
    }
    TPQ_STAMP(7);
}

// out = epilogue(sum over the splits), element by element
template <class Epilogue>
__global__ __launch_bounds__(256) void ternary_slab_finish_kernel(const int32_t* __restrict__ partial, int splits, int M, int N, Epilogue ep) {
    const int64_t total = static_cast<int64_t>(M) * N;
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total; idx += gridDim.x * 256ll) {
        int v = 0;
        for (int s = 0; s < splits; ++s) v += partial[s * total + idx];
        const int m = static_cast<int>(idx / N), n = static_cast<int>(idx - static_cast<int64_t>(m) * N);
        ep.store_scaled(idx, v, ep.row_scale_of(m), ep.bias_of(n));
    }
}

// Splits of K for the slab kernel (1: no workspace needed); 0 when the kernel does not take the shape.
// It is built for one pass of workgroups over the chip: every 32 rows expand the packed weights again, which the
// tile kernel of ternary_gemm_kernel.h does once per 128 (or 64) rows.  Measured (us, bf16 out, slab / tile kernel):
//   2560 -> 6912: 8.7 / 9.6 at 64 rows, 9.4 / 11.3 at 128, 17.0 / 15.9 at 256
//   6912 -> 2560 (three splits): 10.6 / 16.2 at 64, 12.6 / 16.8 at 128, 23.9 / 20.0 at 256
//   4096 -> 4096 (two splits): 10.5 / 11.4 at 33, 11.1 / 11.7 at 64, 13.3 / 12.4 at 128; 5120 -> 5120: 11.4 / 13.2 at 33,
//   11.9 / 13.4 at 64: with two splits the second kernel that adds them costs what the shorter chain saves once the
//   row tiles fill the chip, so two splits are taken up to 64 rows only
// Letting the splits meet inside the kernel (every workgroup leaves its sums with agent-scope stores and counts itself
// in, the last one adds and finishes) was built and is slower than the second launch at three splits (6912 -> 2560:
// 13.4 against 12.7 us at 128 rows, 11.6 against 10.1 at 33): store acknowledgement, counter and the reads of the
// other sums are three trips to memory in a row, a launch and one trip are less.
inline int ternary_slab_splits(int64_t M, int64_t N, int64_t K, int compute_units = 256) {
    if (M < 33 || K % 128 != 0 || K < 128 || M > 0x7FFFFFFF / 2 || N > 0x7FFFFFFF / 2 || K > 0x7FFFFFFF / 2) return 0;
    const int64_t units = K / 128;
    const int64_t splits = (units + kSlabUnits - 1) / kSlabUnits;
    const int64_t workgroups = ((M + kSlabRows - 1) / kSlabRows) * ((N + kSlabChannels - 1) / kSlabChannels) * splits;
    if (workgroups > compute_units || (splits == 2 && M > 64) || splits > 8) return 0;
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
    const size_t smem = main_bytes + kSlabRows * sizeof(int);
    auto kernel = ternary_slab_kernel<Epilogue>;
    static std::atomic<uint64_t> configured{0};  // per instantiation
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), static_cast<size_t>(kSlabRows) * kSlabUnits * 128 + kSlabRows * sizeof(int), configured, "ternary slab")) return rc;
    const int64_t n_tiles = (N + kSlabChannels - 1) / kSlabChannels, m_tiles = (M + kSlabRows - 1) / kSlabRows;
    const int64_t gx = 8 * m_tiles * ((n_tiles * splits + 7) / 8);
    TPQ_REQUIRE(gx <= 0x7FFFFFFF, TPQ_ERR_INVALID_VALUE, "ternary slab: shape too large");
    kernel<<<dim3(static_cast<unsigned>(gx)), kSlabThreads, smem, s>>>(
        x, packed, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), per_split, static_cast<int>(main_bytes),
        static_cast<int>(m_tiles), static_cast<int>(n_tiles), splits, splits > 1 ? partial : nullptr, ep);
    if (int rc = check_launch("tpq_ternary_mm (slab)")) return rc;
    if (splits > 1) {
        const int64_t blocks = (M * N + 255) / 256;
        ternary_slab_finish_kernel<Epilogue><<<static_cast<unsigned>(blocks > 2048 ? 2048 : blocks), 256, 0, s>>>(
            partial, splits, static_cast<int>(M), static_cast<int>(N), ep);
        return check_launch("tpq_ternary_mm (slab, finish)");
    }
    return TPQ_OK;
}

}  // namespace
}  // namespace tpq
