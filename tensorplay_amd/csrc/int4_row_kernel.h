// int4 decode for one to four activation rows, every compute unit streaming its share of the weight.
//
// The packed layout keeps the k-tiles of one tile of eight output channels adjacent: tile nT is
// K/32 x 128 bytes = K/256 blocks of 1 KB.  A workgroup of 16 wavefronts takes one tile per round; wavefront w
// reads block w (and w + 16, ... for K > 4096) of it with ONE load, lane l fetching the 16 bytes of channel l%8 in
// k-tile l/8 of the block, so every wavefront load is 1 KB contiguous and a workgroup reads its tile as one
// contiguous run.  Tiles are dealt round-robin over the workgroups, one workgroup per compute unit, so all
// compute units stream the same number of bytes (+- one tile), and the loads of all rounds are issued before the
// first one is looked at.
//
// A wavefront meets the same 256 k in every round, so a lane's 32 activations (16 words) are loaded once and stay
// in registers, together with the two sums the offset correction needs; there is no LDS traffic and no scalar
// traffic for the activations.  Per load and lane: 16 v_and_or_b32 (+ 4 shifts) turn the nibbles into 16-bit float
// pairs (magic + code), 16 v_dot2 multiply them with the activation pairs, and the lane's group parameters fold
// the sum in fp32:   y_lane = scale * (p - corr) + zero * sx,   corr = sum x (magic + 8),  sx = sum x.
// The eight k-tile groups of a wavefront are added with a DPP rotation and two lane-row swaps, the wavefronts of the
// workgroup through LDS, in a fixed order.
//
// The (scale, zero) words of four neighbouring tiles share a 128-byte line per group: the tile order gives those
// four tiles to workgroups of the same XCD (workgroup id mod 8) in the same round, so the line is fetched into one L2.
#pragma once

#include "int4_lane.h"

namespace tpq {
namespace {

constexpr int kRowWaves = 16;    // wavefronts per workgroup

// Sum over the eight lanes l, l ^ 8, l ^ 16, ... (same l % 8), left in all of them, without the LDS crossbar:
// a rotation by 8 inside each row of 16 lanes (DPP), then the swaps of neighbouring rows and of the two halves
// of the wavefront (v_permlane16_swap / v_permlane32_swap: after the swap one register holds the even rows
// twice and the other the odd rows twice, so their sum is the sum of the pair in both places).
__device__ __forceinline__ float lane_group8_sum(float t) {
    int ti = __builtin_bit_cast(int, t);
    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, ti, 0x128 /* row_ror:8 */, 0xF, 0xF, false));
    ti = __builtin_bit_cast(int, t);
    const auto rows = __builtin_amdgcn_permlane16_swap(ti, ti, false, false);
    t = __builtin_bit_cast(float, static_cast<int>(rows[0])) + __builtin_bit_cast(float, static_cast<int>(rows[1]));
    ti = __builtin_bit_cast(int, t);
    const auto halves = __builtin_amdgcn_permlane32_swap(ti, ti, false, false);
    return __builtin_bit_cast(float, static_cast<int>(halves[0])) + __builtin_bit_cast(float, static_cast<int>(halves[1]));
}

// x: [MROWS][K] 16-bit floats; packed: [n_tiles][k_super][8] uint4; sz: [K/group][N] words (scale, zero);
// k_super % 8 == 0 (K % 256 == 0); SEG = ceil(K / 256 / 16) blocks per wavefront and tile; a group is 32 << group_shift k;
// ROUNDS = tiles per workgroup whose loads are in flight together.
template <int DT, int MROWS, int SEG, int ROUNDS>
__global__ __launch_bounds__(kRowWaves* kWave) void int4_row_kernel(const uint16_t* __restrict__ x, const uint4* __restrict__ packed,
                                                                   const uint32_t* __restrict__ sz, uint16_t* __restrict__ y,
                                                                   int N, int K, int n_tiles, int group_shift) {
    using L = Lane16<DT>;
    __shared__ float red[ROUNDS][kRowWaves][MROWS][8];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;  // ceil(blocks per tile / SEG), at most kRowWaves
    const int kt_in_block = lane >> 3, r = lane & 7;
    const int k_super = K >> 5, blocks_per_tile = K >> 8;

    // tile of round `round`: groups of four neighbouring tiles go to four workgroups of one XCD
    const int groups_total = gridDim.x >> 2;  // gridDim.x is a multiple of 32
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    auto tile_of = [&](int round) { return 4 * (xcd + 8 * (local >> 2) + groups_total * round) + (local & 3); };

    // ---- this lane's activations: 32 k per segment, loaded once; zeros for a segment past the end of K ------------
    // (the kernel is free of branches from here to the barrier: a branch makes the compiler wait for every
    // outstanding load at the join, which would serialise the rounds)
    uint32_t xw[SEG][MROWS][16];
    int kb_of[SEG];
    bool seg_live[SEG];
#pragma unroll
    for (int s = 0; s < SEG; ++s) {
        const int kb = wave + s * waves;
        seg_live[s] = kb < blocks_per_tile;          // wave-uniform
        kb_of[s] = seg_live[s] ? kb : 0;             // a dead segment re-reads block 0 against zero activations
        const int k0 = (kb_of[s] * 8 + kt_in_block) * 32;
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
            const uint4* xp = reinterpret_cast<const uint4*>(x + static_cast<size_t>(m) * K + k0);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint4 v = xp[q];
                xw[s][m][4 * q] = v.x; xw[s][m][4 * q + 1] = v.y; xw[s][m][4 * q + 2] = v.z; xw[s][m][4 * q + 3] = v.w;
            }
        }
    }

    uint32_t magic_even, magic_odd;  // kept in VGPRs: v_and_or_b32 takes one scalar operand only
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_even) : "s"(L::kMagicEven));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_odd) : "s"(L::kMagicOdd));

    uint4 q[ROUNDS][SEG];
    uint32_t p[ROUNDS][SEG];
    // every load of ROUNDS rounds before any use; a round past the last tile re-reads the last tile, its sums are dropped
    // The small (scale, zero) loads go first and the order is pinned: loads return in issue order, so a parameter
    // word requested after the weights would hold the first round back until every weight load has landed.
    auto issue = [&](int base) {
        int t[ROUNDS];
#pragma unroll
        for (int u = 0; u < ROUNDS; ++u) {
            const int tile = tile_of(base + u);
            t[u] = tile < n_tiles ? tile : n_tiles - 1;
        }
#pragma unroll
        for (int u = 0; u < ROUNDS; ++u)
#pragma unroll
            for (int s = 0; s < SEG; ++s) {
                const int g = (kb_of[s] * 8 + kt_in_block) >> group_shift;
                p[u][s] = sz[static_cast<size_t>(g) * N + t[u] * 8 + r];  // plain load: the line serves four tiles of this XCD
            }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < ROUNDS; ++u)
#pragma unroll
            for (int s = 0; s < SEG; ++s)
                q[u][s] = nt_load(packed + (static_cast<size_t>(t[u]) * k_super + kb_of[s] * 8) * 8 + lane);
        __builtin_amdgcn_sched_barrier(0);
    };
    issue(0);  // before the first use of the activations: nothing may wait for x ahead of the weight requests

    // the correction terms, while the weights are on their way
    float corr[SEG][MROWS], sx[SEG][MROWS];
#pragma unroll
    for (int s = 0; s < SEG; ++s)
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
#pragma unroll
            for (int w = 0; w < 16; ++w) xw[s][m][w] = seg_live[s] ? xw[s][m][w] : 0u;
            float even = 0.0f, odd = 0.0f;  // words 4j .. 4j+3 pair with magic_even for j = 0, 2
#pragma unroll
            for (int w = 0; w < 16; ++w) {
                if (((w >> 2) & 1) == 0) even = L::dot(xw[s][m][w], L::kOnes, even);
                else odd = L::dot(xw[s][m][w], L::kOnes, odd);
            }
            corr[s][m] = __builtin_fmaf(L::kOffsetEven, even, L::kOffsetOdd * odd);
            sx[s][m] = even + odd;
        }

    for (int base = 0;;) {
        // ---- consume in issue order ---------------------------------------------------------------------------
#pragma unroll
        for (int u = 0; u < ROUNDS; ++u) {
            float yl[MROWS];
#pragma unroll
            for (int m = 0; m < MROWS; ++m) yl[m] = 0.0f;
#pragma unroll
            for (int s = 0; s < SEG; ++s) {
                const uint32_t wq[4] = {q[u][s].x, q[u][s].y, q[u][s].z, q[u][s].w};
                uint32_t v[4][4];
#pragma unroll
                for (int t4 = 0; t4 < 4; ++t4) L::template unpack<false>(wq[t4], v[t4], magic_even, magic_odd);
                const float scale = L::lo(p[u][s]), zero = L::hi(p[u][s]);
#pragma unroll
                for (int m = 0; m < MROWS; ++m) {
                    float part = 0.0f;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int t4 = 0; t4 < 4; ++t4) part = L::dot(xw[s][m][t4 + 4 * j], v[t4][j], part);
                    yl[m] = __builtin_fmaf(scale, part - corr[s][m], yl[m]);
                    yl[m] = __builtin_fmaf(zero, sx[s][m], yl[m]);
                }
            }
#pragma unroll
            for (int m = 0; m < MROWS; ++m) {
                float t = yl[m];
                t = lane_group8_sum(t);
                red[u][wave][m][r] = t;  // the eight lane groups hold the same sums: same value to the same address
            }
        }
        __syncthreads();
        // ---- the wavefronts' partial sums, in wavefront order ------------------------------------------------
        const int tid = threadIdx.x;
        if (tid < ROUNDS * MROWS * 8) {
            const int u = tid / (MROWS * 8), m = (tid / 8) % MROWS, rr = tid & 7;
            const int tile = tile_of(base + u);
            if (tile < n_tiles) {
                float s = 0.0f;
                for (int w = 0; w < waves; ++w) s += red[u][w][m][rr];
                y[static_cast<size_t>(m) * N + tile * 8 + rr] = L::out(s);
            }
        }
        base += ROUNDS;
        if (tile_of(base) >= n_tiles) break;  // workgroup-uniform
        __syncthreads();                      // red is reused by the next batch of rounds
        issue(base);
    }
}

}  // namespace
}  // namespace tpq
