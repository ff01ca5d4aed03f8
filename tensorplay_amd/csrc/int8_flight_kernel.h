// int8 x int8 product for 3..32 activation rows (decode batches of the dynamic int8 linear), every load of a
// wavefront in flight at once: the structure of int4_mfma_flight_kernel.h with int8 operands on both sides.
//
// v_mfma_i32_16x16x64_i8 with the weights as A: lane (i, q) owns weight row n0 + 16 b + i and, in a step of 128 k, the
// 32 bytes at k = 128 s + 32 q (two 16-byte loads = two MFMAs, no conversion).  A workgroup is 16 wavefronts and NB
// blocks of 16 channels; wavefront w owns the steps w, w + 16, ... and requests all of them up front in straight-line
// code: the activations first, as contiguous runs (a wavefront load = eight rows x 128 bytes), staged in a
// wavefront-private LDS tile with rows 144 bytes apart from which lane (m, q) reads its 32 bytes, then the weights in
// the order of their use.  Integer sums: the result does not depend on how the steps are dealt out.  The wavefronts'
// sums meet in LDS; wavefront b finishes block b and stores runs of four channels with the scales fetched first.
#pragma once

#include "int4_mfma_flight_kernel.h"
#include "int8_gemm_kernel.h"

namespace tpq {
namespace {

constexpr int kI8FlightRowStride = 144;  // bytes between the rows of an activation tile in LDS (128 + 16)

template <int XR>
constexpr int i8_flight_resident_steps() { return XR >= 16 ? 1 : 2; }

template <int NB, int MB, int XR>
constexpr size_t i8_flight_lds_bytes() {
    return static_cast<size_t>(kFlightWaves) * i8_flight_resident_steps<XR>() * XR * kI8FlightRowStride  // activation tiles
         + static_cast<size_t>(kFlightWaves) * NB * MB * 4 * kWave * 4;                                 // partial sums
}

// x: [M][K] int8, M <= XR; w: [N][K] int8; K % 128 == 0, 16 <= K / 128 <= 16 SPW and K / 128 > 16 (SPW - 1);
// XR = 8 (MB = 1), 16 (MB = 1) or 32 (MB = 2) rows through LDS
template <int NB, int MB, int SPW, int XR, class Epilogue>
__global__ __launch_bounds__(kFlightWaves* kWave) void int8_flight_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ w, int M,
                                                                         int N, int K, Epilogue ep) {
    static_assert((XR == 8 && MB == 1) || XR == 16 * MB, "rows through LDS: 8, 16 or 32");
    constexpr int XS = i8_flight_resident_steps<XR>();
    extern __shared__ __align__(16) unsigned char flight_lds[];
    unsigned char* const xbuf = flight_lds;
    int* const red = reinterpret_cast<int*>(flight_lds + static_cast<size_t>(kFlightWaves) * XS * XR * kI8FlightRowStride);  // [wave][NB MB][4][64]

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int steps = K / 128;
    const int n0 = blockIdx.x * (16 * NB);

    // this wavefront's steps; a step past the end (last one only) re-reads the wavefront's first step and is not computed
    int step_of[SPW];
#pragma unroll
    for (int j = 0; j < SPW; ++j) {
        const int s = wave + j * kFlightWaves;
        step_of[j] = s < steps ? s : wave;
    }
    const bool last_live = wave + (SPW - 1) * kFlightWaves < steps;

    // ---- requests: activations (lane: row lane / 8 of the run, 16-byte piece lane % 8), then weights -----------
    uint4 xg[SPW][XR / 8];
#pragma unroll
    for (int t = 0; t < XR / 8; ++t) {
        int row = 8 * t + (lane >> 3);
        row = row < M ? row : M - 1;
        const GlobalWords4 src = opaque4(reinterpret_cast<const uint4*>(x + static_cast<size_t>(row) * K) + (lane & 7));
#pragma unroll
        for (int j = 0; j < SPW; ++j) xg[j][t] = as_uint4(src[step_of[j] * 8]);
    }
    order_fence();
    uint4 wq[SPW][NB][2];
    {
        GlobalWords4 w_base[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int n = n0 + 16 * b + i;
            w_base[b] = opaque4(reinterpret_cast<const uint4*>(w + static_cast<size_t>(n < N ? n : N - 1) * K) + q * 2);  // channels past N: a valid row, result dropped
        }
#pragma unroll
        for (int j = 0; j < SPW; ++j)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                wq[j][b][0] = as_uint4(__builtin_nontemporal_load(w_base[b] + step_of[j] * 8));
                wq[j][b][1] = as_uint4(__builtin_nontemporal_load(w_base[b] + step_of[j] * 8 + 1));
                order_fence();
            }
    }

    unsigned char* const my_x = xbuf + static_cast<size_t>(wave) * XS * XR * kI8FlightRowStride;
    v4i d[NB][MB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < MB; ++r) d[b][r] = v4i{0, 0, 0, 0};

    auto compute = [&](int j) {
        v4i xb[MB][2];  // lane (m, q): the 32 bytes of row 16 r + m (mod XR) at k = 128 s + 32 q
#pragma unroll
        for (int r = 0; r < MB; ++r) {
            const unsigned char* xrow = my_x + ((j % XS) * XR + ((16 * r + i) & (XR - 1))) * kI8FlightRowStride + q * 32;
            xb[r][0] = *reinterpret_cast<const v4i*>(xrow);
            xb[r][1] = *reinterpret_cast<const v4i*>(xrow + 16);
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            // the weights enter the step here, not earlier (see the int4 kernel)
            asm volatile("" : "+v"(wq[j][b][0].x), "+v"(wq[j][b][0].y), "+v"(wq[j][b][0].z), "+v"(wq[j][b][0].w), "+v"(wq[j][b][1].x),
                         "+v"(wq[j][b][1].y), "+v"(wq[j][b][1].z), "+v"(wq[j][b][1].w)::"memory");
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int r = 0; r < MB; ++r)
                    d[b][r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, wq[j][b][h]), xb[r][h], d[b][r], 0, 0, 0);
        }
    };

#pragma unroll
    for (int j0 = 0; j0 < SPW; j0 += XS) {
#pragma unroll
        for (int j = j0; j < j0 + XS && j < SPW; ++j)
#pragma unroll
            for (int t = 0; t < XR / 8; ++t)
                *reinterpret_cast<uint4*>(my_x + ((j % XS) * XR + 8 * t + (lane >> 3)) * kI8FlightRowStride + (lane & 7) * 16) = xg[j][t];
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = j0; j < j0 + XS && j < SPW; ++j) {
            if (j < SPW - 1) {
                compute(j);
            } else if (last_live) {  // wave-uniform, after every request
                compute(j);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_wave_barrier();
    }

    // ---- the wavefronts' partial sums ------------------------------------------------------------------------
    // wavefront t finishes output block t (channel block t / MB, row block t % MB): lane (m, q) stores row 16 r + m,
    // channels n0 + 16 b + 4 q .. + 3.  Its scales are asked for here, ahead of the exchange: behind it they are a
    // trip to memory that nothing covers.
    static_assert(NB * MB <= kFlightWaves, "one output block per finishing wavefront");
    const int fin_m = 16 * (wave % MB) + i, fin_n = n0 + 16 * (wave / MB) + 4 * q;
    const bool finishes = wave < NB * MB && fin_m < M && fin_n < N;
    float row_scale = 0.0f, col_scale[4] = {0.0f, 0.0f, 0.0f, 0.0f}, bias_n[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (finishes) {
        row_scale = ep.row_scale_of(fin_m);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int n = fin_n + v < N ? fin_n + v : fin_n;
            col_scale[v] = ep.col_scale_of(n);
            bias_n[v] = ep.bias_of(n);
        }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[((wave * NB * MB + b * MB + r) * 4 + v) * kWave + lane] = d[b][r][v];
    __syncthreads();
    if (finishes) {
        const int t = wave;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            int sum = 0;
#pragma unroll
            for (int ww = 0; ww < kFlightWaves; ++ww) sum += red[((ww * NB * MB + t) * 4 + v) * kWave + lane];
            if (fin_n + v < N) ep.store_scaled(static_cast<int64_t>(fin_m) * N + fin_n + v, sum, row_scale, col_scale[v], bias_n[v]);
        }
    }
}

}  // namespace
}  // namespace tpq
