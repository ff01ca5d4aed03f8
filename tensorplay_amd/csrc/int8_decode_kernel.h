// int8 x int8 product for a few activation rows (1..16 per launch: decode batches of the dynamic int8
// linear), K % 128 == 0.  At these sizes the product is a stream over the weight, one byte per element,
// and what matters is reading it once at full rate: v_mfma_i32_16x16x64_i8 with the WEIGHTS as the A
// operand, exactly as the weight-only decode kernels do.  Lane (i, q) owns weight row n0 + i and, in a
// step of 128 k, the 32 bytes at k = 128 s + 32 q: two 16-byte loads, each the A operand of one MFMA
// (which k sits in which slot of the instruction is free as long as both operands agree, and the
// activations are loaded the same way: lane (m, q) takes x[m][128 s + 32 q .. + 32)).  No conversion,
// no LDS staging: the only vector-ALU work is the epilogue.  D comes out as lane (m, q) x channels
// n0 + 4 q + v in int32, exact; the wavefronts of a workgroup take the steps round-robin and add their
// partial sums through LDS.  Columns m >= M stay zero and load nothing.
#pragma once

#include "int8_gemm_kernel.h"

namespace tpq {
namespace {

template <int WAVES, class Epilogue>
__global__ __launch_bounds__(WAVES * kWave) void int8_decode_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ w,
                                                                   int M, int N, int K, Epilogue ep) {
    __shared__ int red[WAVES][4][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int steps = K / 128;
    const int n0 = blockIdx.x * 16;
    const int n_row = n0 + i < N ? n0 + i : N - 1;  // rows past N: a valid row, result dropped
    const bool row_live = i < M;
    const uint4* w_base = reinterpret_cast<const uint4*>(w + static_cast<size_t>(n_row) * K) + q * 2;
    const uint4* x_base = reinterpret_cast<const uint4*>(x + static_cast<size_t>(row_live ? i : 0) * K) + q * 2;

    struct Step {
        uint4 w[2];
        uint4 xv[2];
    };
    auto load = [&](int s, Step& st) {
        st.w[0] = nt_load(w_base + s * 8);
        st.w[1] = nt_load(w_base + s * 8 + 1);
        if (row_live) {
            st.xv[0] = x_base[s * 8];
            st.xv[1] = x_base[s * 8 + 1];
        }
    };
    v4i d0 = {0, 0, 0, 0}, d1 = {0, 0, 0, 0};  // two accumulators taking turns
    auto compute = [&](const Step& st) {
        d0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, st.w[0]), __builtin_bit_cast(v4i, st.xv[0]), d0, 0, 0, 0);
        d1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, st.w[1]), __builtin_bit_cast(v4i, st.xv[1]), d1, 0, 0, 0);
    };

    // this wavefront's steps: wave, wave + WAVES, ...; four in flight (a step is 64 bytes per lane)
    constexpr int kRing = 4;
    Step ring[kRing] = {};
#pragma unroll
    for (int r = 0; r < kRing; ++r)
        if (wave + r * WAVES < steps) load(wave + r * WAVES, ring[r]);
    for (int base = wave; base < steps; base += kRing * WAVES) {
#pragma unroll
        for (int r = 0; r < kRing; ++r) {
            const int s = base + r * WAVES;
            if (s < steps) {
                compute(ring[r]);
                if (s + kRing * WAVES < steps) load(s + kRing * WAVES, ring[r]);
            }
        }
    }

#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][v][lane] = d0[v] + d1[v];
    __syncthreads();
    if (wave == 0 && row_live) {  // lane (m, q): channels n0 + 4 q + v
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            int sum = 0;
#pragma unroll
            for (int ww = 0; ww < WAVES; ++ww) sum += red[ww][v][lane];
            const int n = n0 + 4 * q + v;
            if (n < N) ep.store(static_cast<int64_t>(i) * N + n, i, n, sum);
        }
    }
}

inline bool int8_decode_ok(const void* a, const void* w, int64_t M, int64_t N, int64_t K) {
    return M >= 1 && K >= 128 && K % 128 == 0 && aligned(a, 16) && aligned(w, 16) && N <= 0x7FFFFFF0 && K <= 0x7FFFFF80;
}

// slabs of 16 rows; the epilogue sees row indices of the whole problem through `rebase`
template <class Epilogue, class Rebase>
int launch_int8_decode(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Epilogue ep, Rebase rebase, hipStream_t s) {
    const int steps = static_cast<int>(K / 128);
    for (int64_t m0 = 0; m0 < M; m0 += 16) {
        const int rows = static_cast<int>(M - m0 < 16 ? M - m0 : 16);
        const dim3 grid(static_cast<unsigned>((N + 15) / 16));
        const Epilogue slab = rebase(ep, m0);
        if (steps >= 32)
            int8_decode_kernel<8, Epilogue><<<grid, 8 * kWave, 0, s>>>(a + m0 * K, w, rows, static_cast<int>(N), static_cast<int>(K), slab);
        else
            int8_decode_kernel<4, Epilogue><<<grid, 4 * kWave, 0, s>>>(a + m0 * K, w, rows, static_cast<int>(N), static_cast<int>(K), slab);
    }
    return check_launch("int8 decode gemm");
}

}  // namespace
}  // namespace tpq
