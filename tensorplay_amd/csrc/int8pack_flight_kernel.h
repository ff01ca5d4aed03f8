// int8 weight-only decode for 3..16 activation rows (fp16 / bf16) on the matrix cores, every load of a wavefront in
// flight at once: the structure of int4_mfma_flight_kernel.h at one byte per weight.
//
// A workgroup is 16 wavefronts and NB blocks of 16 output channels; wavefront w owns the steps (128 k) w, w + 16, ...
// and requests them all before the first use, in straight-line code: first the activations as contiguous row runs
// (only the XR rows that can be live, staged in a wavefront-private LDS tile, see the int4 kernel), then the weights
// in the order of their use: lane (i, q) owns row n0 + 16 b + i and the 32 bytes at k = 128 s + 32 q, two 16-byte
// loads, whole 128-byte lines per row and step.  Every dword (four int8) becomes two 16-bit float pairs exactly as in
// int8pack_mfma_kernel (fp16: xor 0x80808080, v_perm_b32 next to the exponent byte 0x64, one packed subtract of 1152;
// bf16: a sign-extending byte-to-float conversion per code); the products are exact, accumulate in fp32 over the
// wavefront's steps, the wavefronts' sums are added in wavefront order and the per-channel scale multiplies the total
// (reference: _weight_int8pack_mm, p10/src/backend/cuda/QuantGemmKernels.cu:339-405).
#pragma once

#include "int4_mfma_flight_kernel.h"

namespace tpq {
namespace {

template <int NB, int SPW, int XR>
constexpr size_t int8_flight_lds_bytes() {
    return static_cast<size_t>(kFlightWaves) * flight_resident_steps<XR>() * XR * kFlightRowStride  // activation tiles
         + static_cast<size_t>(kFlightWaves) * NB * 4 * (4 * XR) * 4;                                // partial sums, live rows
}

// x: [M][K] 16-bit, M <= XR; w: [N][K] int8; scale: [N]; y: [M][N]; K % 128 == 0, 16 <= K / 128 <= 16 SPW and
// K / 128 > 16 (SPW - 1)
// RB = 2 (XR = 16): 17..32 rows as two blocks of 16 against the same weight registers, as in the int4 kernel.
template <int DT, int NB, int SPW, int XR, int RB = 1>
__global__ __launch_bounds__(kFlightWaves* kWave) void int8pack_flight_kernel(const uint16_t* __restrict__ x, const int8_t* __restrict__ w,
                                                                             const float* __restrict__ scale, uint16_t* __restrict__ y,
                                                                             int M, int N, int K) {
    static_assert(XR == 4 || XR == 8 || XR == 16, "rows through LDS: 4, 8 or 16");
    static_assert(RB == 1 || (RB == 2 && XR == 16), "two row blocks: 16 rows each");
    constexpr int XS = flight_resident_steps<XR>();
    extern __shared__ __align__(16) unsigned char flight_lds[];
    unsigned char* const xbuf = flight_lds;
    float* const red = reinterpret_cast<float*>(flight_lds + static_cast<size_t>(kFlightWaves) * XS * XR * kFlightRowStride);  // [wave][NB][4][4 XR]

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

    // ---- requests: activations, then weights --------------------------------------------------------------
    uint4 xg[SPW][XR / 4];
#pragma unroll
    for (int t = 0; t < XR / 4; ++t) {
        int row = 4 * t + q;
        row = row < M ? row : M - 1;
        const GlobalWords4 src = opaque4(reinterpret_cast<const uint4*>(x + static_cast<size_t>(row) * K) + i);
#pragma unroll
        for (int j = 0; j < SPW; ++j) xg[j][t] = as_uint4(src[step_of[j] * 16]);
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

    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 bias = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
    uint32_t magic;  // exponent bytes, kept in a VGPR behind an opaque move
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "s"(0x64646464u));

    unsigned char* const my_x = xbuf + static_cast<size_t>(wave) * XS * XR * kFlightRowStride;
    float4_t d[RB][NB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int b = 0; b < NB; ++b) d[rb][b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    auto compute = [&](int j, int rb) {
        // lane (m, q): the 64 bytes of row m % XR at k = 128 s + 32 q; MFMA u takes bytes 16 u .. 16 u + 15 of them
        word4_t xb[4];
        const unsigned char* xrow = my_x + ((j % XS) * XR + (i & (XR - 1))) * kFlightRowStride + q * 64;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint4 v = *reinterpret_cast<const uint4*>(xrow + u * 16);
            xb[u] = word4_t{v.x, v.y, v.z, v.w};
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            // the weights enter the step here, not earlier (see the int4 kernel)
            asm volatile("" : "+v"(wq[j][b][0].x), "+v"(wq[j][b][0].y), "+v"(wq[j][b][0].z), "+v"(wq[j][b][0].w), "+v"(wq[j][b][1].x),
                         "+v"(wq[j][b][1].y), "+v"(wq[j][b][1].z), "+v"(wq[j][b][1].w)::"memory");
#pragma unroll
            for (int u = 0; u < 4; ++u) {  // MFMA u (16x16x32): k = 8 u .. 8 u + 7 of the lane's 32
                uint32_t a[4];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t word = dword_of(wq[j][b][u >> 1], (2 * u + h) & 3);
                    if constexpr (DT == TPQ_DTYPE_F16) {
                        const uint32_t t = word ^ 0x80808080u;
                        const uint32_t lo = __builtin_amdgcn_perm(magic, t, 0x04010400u);  // (1152 + b0, 1152 + b1)
                        const uint32_t hi = __builtin_amdgcn_perm(magic, t, 0x04030402u);  // (1152 + b2, 1152 + b3)
                        a[2 * h] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, lo) - bias);
                        a[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, hi) - bias);
                    } else {
                        uint32_t f[4];  // bf16 is the upper half of a float and an int8 has eight significant bits: exact
#pragma unroll
                        for (int e = 0; e < 4; ++e) f[e] = __builtin_bit_cast(uint32_t, static_cast<float>(static_cast<int8_t>(word >> (8 * e))));
                        a[2 * h] = __builtin_amdgcn_perm(f[1], f[0], 0x07060302u);
                        a[2 * h + 1] = __builtin_amdgcn_perm(f[3], f[2], 0x07060302u);
                    }
                }
                d[rb][b] = MfmaLane<DT>::mfma(word4_t{a[0], a[1], a[2], a[3]}, xb[u], d[rb][b]);
            }
        }
    };

#pragma unroll
    for (int j0 = 0; j0 < SPW; j0 += XS) {
#pragma unroll
        for (int j = j0; j < j0 + XS && j < SPW; ++j)
#pragma unroll
            for (int t = 0; t < XR / 4; ++t)
                *reinterpret_cast<uint4*>(my_x + ((j % XS) * XR + 4 * t + q) * kFlightRowStride + i * 16) = xg[j][t];
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (RB == 2) {  // XS = 1: step j0 of the first block is in LDS, its registers take the second block's
            order_fence();
#pragma unroll
            for (int t = 0; t < XR / 4; ++t) {
                int row = XR + 4 * t + q;
                row = row < M ? row : M - 1;
                const GlobalWords4 src = opaque4(reinterpret_cast<const uint4*>(x + static_cast<size_t>(row) * K) + i);
                xg[j0][t] = as_uint4(src[step_of[j0] * 16]);
            }
            order_fence();
        }
#pragma unroll
        for (int j = j0; j < j0 + XS && j < SPW; ++j) {
            if (j < SPW - 1) {
                compute(j, 0);
            } else if (last_live) {  // wave-uniform, after every request
                compute(j, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_wave_barrier();
    }
    if constexpr (RB == 2) {
        static_assert(RB == 1 || XS == 1, "the second block's requests go step by step");
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
#pragma unroll
            for (int t = 0; t < XR / 4; ++t) *reinterpret_cast<uint4*>(my_x + (4 * t + q) * kFlightRowStride + i * 16) = xg[j][t];
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_sched_barrier(0);
            if (j < SPW - 1) {
                compute(j, 1);
            } else if (last_live) {
                compute(j, 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_wave_barrier();
        }
    }

    // ---- the wavefronts' partial sums, added in wavefront order -----------------------------------------------
    // wavefront w finishes block w: lane (m, q) stores row m, channels n0 + 16 w + 4 q + v; their scales are asked for
    // ahead of the exchange
    static_assert(NB <= kFlightWaves, "one block per finishing wavefront");
    float scale_n[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (wave < NB) {
        const auto sp = pinned_global(scale);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int n = n0 + 16 * wave + 4 * q + v;
            scale_n[v] = sp[n < N ? n : N - 1];
        }
    }
    const int slot = q * XR + i;  // live lanes (rows < XR) only
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        if (rb > 0) __syncthreads();  // the sums of the first block have been read
        if (i < XR) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int v = 0; v < 4; ++v) red[((wave * NB + b) * 4 + v) * (4 * XR) + slot] = d[rb][b][v];
        }
        __syncthreads();
        const int out_row = XR * rb + i;
        // wavefront w finishes block w: lane (m, q) stores row m, channels n0 + 16 b + 4 q + v
        for (int b = wave; b < NB; b += kFlightWaves) {
            if (i >= XR || out_row >= M) continue;
            const int n = n0 + 16 * b + 4 * q;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float sum = 0.0f;
#pragma unroll
                for (int ww = 0; ww < kFlightWaves; ++ww) sum += red[((ww * NB + b) * 4 + v) * (4 * XR) + slot];
                if (n + v < N) y[static_cast<size_t>(out_row) * N + n + v] = Elem<DT>::store(__fmul_rn(sum, scale_n[v]));
            }
        }
    }
}

}  // namespace
}  // namespace tpq
