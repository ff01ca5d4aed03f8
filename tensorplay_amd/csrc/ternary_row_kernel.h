// Ternary-weight product for ONE activation row (the decode step of the BitNet linear), K % 64 == 0, K <= 8192.
//
// The matrix-core kernel of ternary_decode_mfma.h asks for the packed weights in the MFMA's operand order: a wave-level
// load takes 64 bytes out of each of 16 rows, and the activations are fetched per lane.  The vector memory path takes a
// wave-level load at a price per cache line it touches, not per byte, so at one row (where the matrix cores have
// nothing to amortise) that order costs more than the arithmetic.  Here the packed matrix is read as what it is in
// memory, a flat run of bytes:
//   * a workgroup owns `rows_wg` consecutive channels = rows_wg * K / 4 contiguous bytes, one 16-byte chunk (64 codes)
//     per thread, so every wave-level load is 1 KB of whole lines and every wavefront of the chip has exactly one;
//   * the activation row is read once per workgroup, contiguously, ahead of the weights (loads return in order), brought
//     into the field order of the packed bytes by a 4 x 4 byte transpose and parked in LDS (K bytes); an LDS-only
//     barrier, so that nobody waits for its weights in front of it;
//   * (w << 2 f) & 0xC0C0C0C0 puts field f of four packed bytes at the top of its byte: 64 x code as a signed byte; one
//     v_dot4_i32_i8 with the four activations of that field position, 3 instructions per 4 codes, and the 64 leaves the
//     finished sum with an exact shift;
//   * chunk t of the workgroup belongs to channel t / (K / 64): the lanes add their sums to the channel's word in LDS
//     (ds_add_u32), the first rows_wg threads scale, round and store.
// Exact int32 sums, the same as every other ternary kernel here.
#pragma once

#include "int8_gemm_kernel.h"
#include "ternary_decode_mfma.h"

namespace tpq {
namespace {

constexpr int kTernaryRowMaxK = 8192;
constexpr int kTernaryRowMaxThreads = 1024;
__host__ __device__ constexpr int ternary_row_x_slots(int K) { return (K >> 4) + (K >> 8) + 1; }  // 16-byte slots of the parked activations

// grid: ceil(N / rows_wg); block: 64 * ceil(rows_wg * K / 64 / 64) threads >= K / 16; LDS: 16 ternary_row_x_slots(K) + 4 rows_wg bytes
template <class Epilogue>
__global__ __launch_bounds__(kTernaryRowMaxThreads) void ternary_row_kernel(const int8_t* __restrict__ x, const uint8_t* __restrict__ packed, int N,
                                                                           int K, int rows_wg, float inv_chunks_per_row, Epilogue ep) {
    // [K / 16 + K / 256]: slot 4 c + d + c / 4 holds the transposed piece d of chunk c (one slot of padding per four
    // chunks: the sixteen lanes a 16-byte read serves together, chunks c .. c + 15, then hit sixteen different groups of
    // four banks; without it chunks four apart met in the same banks and most of the kernel's LDS cycles were conflicts)
    extern __shared__ uint4 x_fields[];
    int* const sums = reinterpret_cast<int*>(x_fields + ternary_row_x_slots(K));
    const int t = threadIdx.x;
    const int cpr = K >> 6;  // 16-byte chunks in a packed row
    const int row0 = blockIdx.x * rows_wg;
    const int rows_here = N - row0 < rows_wg ? N - row0 : rows_wg;
    const bool live = t < rows_here * cpr;
    const int pieces = K >> 4;

    // requests in the order they are needed (loads come back in the order they were made): activations, weights, bias
    const uint4 xr = reinterpret_cast<const uint4*>(x)[t < pieces ? t : 0];
    const uint4 w = nt_load(reinterpret_cast<const uint4*>(packed + static_cast<size_t>(row0) * (static_cast<size_t>(K) >> 2)) + (live ? t : 0));
    const float row_scale = ep.row_scale_of(0);
    const int n = row0 + (t < rows_here ? t : 0);
    const bool with_bias = ep.out && ep.bias;
    const float bias_raw = *(with_bias ? ep.bias + n : reinterpret_cast<const float*>(x));  // no branch around a load: some readable word instead

    if (t < rows_wg) sums[t] = 0;
    if (t < pieces) {
        const v4i f = transpose_4x4_bytes(xr);
        const int c = t >> 2, d = t & 3;
        x_fields[4 * c + d + (c >> 2)] = make_uint4(static_cast<uint32_t>(f[0]), static_cast<uint32_t>(f[1]), static_cast<uint32_t>(f[2]), static_cast<uint32_t>(f[3]));
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the weights stay in flight

    const int row = static_cast<int>((static_cast<float>(t) + 0.5f) * inv_chunks_per_row);  // t / cpr exactly: t < 1024, cpr <= 128
    const int c = t - row * cpr;
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
    int acc = 0;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint4 xf = x_fields[4 * c + d + (c >> 2)];
        const uint32_t fields[4] = {xf.x, xf.y, xf.z, xf.w};
#pragma unroll
        for (int f = 0; f < 4; ++f)
            acc = __builtin_amdgcn_sdot4(static_cast<int>(fields[f]), static_cast<int>((words[d] << (2 * f)) & 0xC0C0C0C0u), acc, false);
    }
    // Up to 128 lanes add to one channel's word, and LDS serves the lanes of one address one after the other: where four
    // (eight) neighbouring chunks always belong to one channel, their lanes add up first and one of them goes to LDS.
    if (!live) acc = 0;
    if ((cpr & 3) == 0) {
        acc += __builtin_amdgcn_mov_dpp(acc, 0xB1, 0xF, 0xF, true);  // quad_perm [1, 0, 3, 2]
        acc += __builtin_amdgcn_mov_dpp(acc, 0x4E, 0xF, 0xF, true);  // quad_perm [2, 3, 0, 1]
        if ((cpr & 7) == 0) {
            acc += __builtin_amdgcn_mov_dpp(acc, 0x141, 0xF, 0xF, true);  // row_half_mirror: the other quad of the eight
            if (live && (t & 7) == 0) __hip_atomic_fetch_add(&sums[row], acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else if (live && (t & 3) == 0) {
            __hip_atomic_fetch_add(&sums[row], acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    } else if (live) {
        __hip_atomic_fetch_add(&sums[row], acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (t < rows_here) ep.store_scaled(n, sums[t] >> 6, row_scale, with_bias ? bias_raw : 0.0f);
}

// rows per workgroup (0: the kernel does not take the shape).  Up to 8 MB of packed weights the wavefronts all fit the
// chip at once (8192 of them): whole rounds of workgroups over the compute units where the channel count allows, at
// most 16 wavefronts and at least the K / 16 threads that park the activations.  Larger weights: four rows, the
// smallest workgroups, so that the rounds of wavefronts follow each other closely.  Measured, weights streamed from HBM
// (us, this kernel / ternary_decode_mfma.h):
//   2560 -> 6912  3.13 / 4.33 (cache-resident 2.60 / 3.79)      6912 -> 2560  3.29 / 4.92 (2.81 / 4.22)
//   2048 x 2048   2.35 / 3.03      4096 x 4096   3.05 / 3.81      5120 x 5120   3.63 / 4.80      4096 -> 11008  4.41 / 5.80
//   5120 -> 13824 6.10 / 7.27      8192 x 8192   5.80 / 7.79      8192 -> 16384 9.25 / 10.24     8192 -> 28672  14.6 / 15.9
//   4096 -> 32000 8.55 / 10.4
// (with every lane adding to the channel's LDS word by itself the kernel lost beyond 8 MB: 8192 x 8192 8.57)
inline int ternary_row_rows_per_workgroup(int64_t M, int64_t N, int64_t K, int compute_units = 256) {
    if (M != 1 || K < 64 || K % 64 != 0 || K > kTernaryRowMaxK || N < 1 || N > 0x7FFFFFF0) return 0;
    const int64_t cpr = K / 64, most = kTernaryRowMaxThreads / cpr;
    if (most < 4) return 0;
    if (const char* e = tuning_env("TPQ_TERNARY_ROW_WG")) {
        const int64_t rows = std::atoll(e);
        return rows >= 4 && rows <= most ? static_cast<int>(rows) : 0;
    }
    if (N * K > (int64_t{1} << 25)) return 4;
    for (int64_t rounds = 1; rounds <= 64; ++rounds) {
        const int64_t rows = (N + compute_units * rounds - 1) / (compute_units * rounds);
        if (rows <= most) return static_cast<int>(rows < 4 ? 4 : rows);
    }
    return static_cast<int>(most);
}

template <class Epilogue>
int launch_ternary_row(const int8_t* x, const uint8_t* packed, int64_t N, int64_t K, int rows_wg, Epilogue ep, hipStream_t s) {
    const int64_t cpr = K / 64, threads = (rows_wg * cpr + 63) / 64 * 64;
    TPQ_REQUIRE(K % 64 == 0 && K <= kTernaryRowMaxK && rows_wg >= 4 && threads <= kTernaryRowMaxThreads && threads >= K / 16 && threads >= rows_wg,
                TPQ_ERR_INVALID_VALUE, "ternary row kernel: workgroup shape");
    const size_t smem = 16 * static_cast<size_t>(ternary_row_x_slots(static_cast<int>(K))) + 4 * static_cast<size_t>(rows_wg);
    ternary_row_kernel<Epilogue><<<static_cast<unsigned>((N + rows_wg - 1) / rows_wg), static_cast<unsigned>(threads), smem, s>>>(
        x, packed, static_cast<int>(N), static_cast<int>(K), rows_wg, 1.0f / static_cast<float>(cpr), ep);
    return check_launch("tpq_ternary_mm (one row)");
}

}  // namespace
}  // namespace tpq
