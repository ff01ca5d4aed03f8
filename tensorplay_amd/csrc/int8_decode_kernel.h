// int8 x int8 product for a few activation rows (1..16 MB per launch: decode batches of the dynamic int8
// linear), K % 128 == 0, NB blocks of 16 channels per workgroup.  At these sizes the product is a stream over the weight, one byte per element,
// and what matters is reading it once at full rate: v_mfma_i32_16x16x64_i8 with the WEIGHTS as the A
// operand, exactly as the weight-only decode kernels do.  Lane (i, q) owns weight row n0 + i and, in a
// step of 128 k, the 32 bytes at k = 128 s + 32 q: two 16-byte loads, each the A operand of one MFMA
// (which k sits in which slot of the instruction is free as long as both operands agree, and the
// activations are loaded the same way: lane (m, q) takes x[m][128 s + 32 q .. + 32)).  No conversion,
// no LDS staging: the only vector-ALU work is the epilogue.  D comes out as lane (m, q) x channels
// n0 + 4 q + v in int32, exact; the wavefronts of a workgroup take the steps round-robin and add their
// partial sums through LDS.  Columns m >= M stay zero and load nothing.
#pragma once

#include <cstdlib>

#include "int8_gemm_kernel.h"
#include "int8_flight_kernel.h"

namespace tpq {
namespace {

template <int NB, int MB, int WAVES, class Epilogue>
__global__ __launch_bounds__(WAVES * kWave) void int8_decode_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ w,
                                                                   int M, int N, int K, Epilogue ep) {
    __shared__ int red[WAVES][NB * MB][4][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int steps = K / 128;
    const int n0 = blockIdx.x * (16 * NB);
    const uint4* w_base[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int n = n0 + 16 * b + i;
        w_base[b] = reinterpret_cast<const uint4*>(w + static_cast<size_t>(n < N ? n : N - 1) * K) + q * 2;  // rows past N: a valid row, result dropped
    }
    bool row_live[MB];
    const uint4* x_base[MB];
#pragma unroll
    for (int r = 0; r < MB; ++r) {
        row_live[r] = 16 * r + i < M;
        x_base[r] = reinterpret_cast<const uint4*>(x + static_cast<size_t>(row_live[r] ? 16 * r + i : 0) * K) + q * 2;
    }

    struct Step {
        uint4 w[NB][2];
        uint4 xv[MB][2];
    };
    auto load = [&](int s, Step& st) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            st.w[b][0] = nt_load(w_base[b] + s * 8);
            st.w[b][1] = nt_load(w_base[b] + s * 8 + 1);
        }
#pragma unroll
        for (int r = 0; r < MB; ++r)
            if (row_live[r]) {
                st.xv[r][0] = x_base[r][s * 8];
                st.xv[r][1] = x_base[r][s * 8 + 1];
            }
    };
    v4i d[NB][MB][2] = {};  // two accumulators per output block taking turns
    auto compute = [&](const Step& st) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int r = 0; r < MB; ++r)
                    d[b][r][h] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, st.w[b][h]), __builtin_bit_cast(v4i, st.xv[r][h]),
                                                                      d[b][r][h], 0, 0, 0);
    };

    // this wavefront's steps: wave, wave + WAVES, ...; RING in flight (a step is 32 (NB + MB) bytes per lane)
    constexpr int kRing = NB + MB >= 4 ? 2 : 4;
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

    // The finishing wavefront asks for its scales and bias values here, ahead of the exchange of the partial sums:
    // fetched element by element in the store loop each is a trip to memory that the next store waits for (a load
    // behind a store to `out` cannot be moved ahead of it).
    float row_scale[MB], col_scale[NB][4], bias_n[NB][4];
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < MB; ++r) row_scale[r] = ep.row_scale_of(row_live[r] ? 16 * r + i : 0);
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int n = n0 + 16 * b + 4 * q + v;
                col_scale[b][v] = ep.col_scale_of(n < N ? n : N - 1);
                bias_n[b][v] = ep.bias_of(n < N ? n : N - 1);
            }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][b * MB + r][v][lane] = d[b][r][0][v] + d[b][r][1][v];
    __syncthreads();
    if (wave == 0) {  // lane (m, q): rows 16 r + m, channels n0 + 16 b + 4 q + v
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int r = 0; r < MB; ++r)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    int sum = 0;
#pragma unroll
                    for (int ww = 0; ww < WAVES; ++ww) sum += red[ww][b * MB + r][v][lane];
                    const int n = n0 + 16 * b + 4 * q + v, m = 16 * r + i;
                    if (row_live[r] && n < N) ep.store_scaled(static_cast<int64_t>(m) * N + n, sum, row_scale[r], col_scale[b][v], bias_n[b][v]);
                }
    }
}

// One to four activation rows: the weight rows are contiguous, so a wavefront reads them directly.  Lane l owns the
// 16 k of chunk 64 t + l of its pass (a pass = four such turns = 4096 k): one 16-byte load per turn and channel (1 KB
// contiguous per wavefront and load) and the 16 bytes of every activation row that go with them, shared by the
// wavefront's four channels; v_dot4_i32_i8 multiplies.  Every load is issued before the first use, so the whole
// weight is requested within the first microsecond.  Workgroup = channel groups x passes; the lanes' sums meet by a
// butterfly, the passes' through LDS; integer sums, so the result does not depend on any of this.
constexpr int kI8RowChannels = 4, kI8RowTurns = 4;

template <int ROWS, int WAVES, class Epilogue>
__global__ __launch_bounds__(WAVES * kWave) void int8_row_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ w, int N, int K,
                                                                int passes, int groups, Epilogue ep) {
    __shared__ int red[WAVES][kI8RowChannels * ROWS];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = wave / passes, pass = wave - g * passes;
    const int n0 = (blockIdx.x * groups + g) * kI8RowChannels;
    const bool active = g < groups && n0 < N;
    // thread = (group, channel, row) finishes one output; its scales are asked for ahead of the weights
    const int tid = threadIdx.x;
    const bool finishes = tid < groups * kI8RowChannels * ROWS;
    const int out_group = tid / (kI8RowChannels * ROWS), out_rem = tid - out_group * (kI8RowChannels * ROWS);
    const int out_c = out_rem / ROWS, out_r = out_rem - out_c * ROWS;
    const int out_n = (blockIdx.x * groups + out_group) * kI8RowChannels + out_c;
    float row_scale = 0.0f, col_scale = 0.0f, bias_n = 0.0f;
    if (finishes && out_n < N) {
        row_scale = ep.row_scale_of(out_r);
        col_scale = ep.col_scale_of(out_n);
        bias_n = ep.bias_of(out_n);
    }
    int acc[kI8RowChannels][ROWS];
#pragma unroll
    for (int c = 0; c < kI8RowChannels; ++c)
#pragma unroll
        for (int r = 0; r < ROWS; ++r) acc[c][r] = 0;
    if (active) {
        const int chunks = K >> 4;
        uint4 wv[kI8RowChannels][kI8RowTurns];
        uint4 xv[ROWS][kI8RowTurns];
#pragma unroll
        for (int t = 0; t < kI8RowTurns; ++t) {
            const int chunk = (pass * kI8RowTurns + t) * kWave + lane;
            const bool live = chunk < chunks;
            const int cl = live ? chunk : chunks - 1;  // past the end: a valid chunk, multiplied by zeros
#pragma unroll
            for (int c = 0; c < kI8RowChannels; ++c) {
                const int n = n0 + c < N ? n0 + c : N - 1;
                wv[c][t] = nt_load(reinterpret_cast<const uint4*>(w + static_cast<size_t>(n) * K) + cl);
            }
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
                xv[r][t] = live ? reinterpret_cast<const uint4*>(x + static_cast<size_t>(r) * K)[cl] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < kI8RowTurns; ++t)
#pragma unroll
            for (int c = 0; c < kI8RowChannels; ++c)
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    int a = acc[c][r];
                    a = __builtin_amdgcn_sdot4(static_cast<int>(xv[r][t].x), static_cast<int>(wv[c][t].x), a, false);
                    a = __builtin_amdgcn_sdot4(static_cast<int>(xv[r][t].y), static_cast<int>(wv[c][t].y), a, false);
                    a = __builtin_amdgcn_sdot4(static_cast<int>(xv[r][t].z), static_cast<int>(wv[c][t].z), a, false);
                    a = __builtin_amdgcn_sdot4(static_cast<int>(xv[r][t].w), static_cast<int>(wv[c][t].w), a, false);
                    acc[c][r] = a;
                }
#pragma unroll
        for (int c = 0; c < kI8RowChannels; ++c)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) acc[c][r] = wave_sum(acc[c][r]);
    }
    if (lane == 0) {
#pragma unroll
        for (int c = 0; c < kI8RowChannels; ++c)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) red[wave][c * ROWS + r] = acc[c][r];
    }
    __syncthreads();
    if (finishes && out_n < N) {
        int sum = 0;
        for (int ps = 0; ps < passes; ++ps) sum += red[out_group * passes + ps][out_rem];
        ep.store_scaled(static_cast<int64_t>(out_r) * N + out_n, sum, row_scale, col_scale, bias_n);
    }
}

// false if the row kernel does not take the shape (rows of more than 32768 k)
template <class Epilogue>
bool launch_int8_rows(const int8_t* a, const int8_t* w, int rows, int64_t N, int64_t K, Epilogue ep, hipStream_t s) {
    const int passes = static_cast<int>((K + 4095) / 4096);
    // small weights need many workgroups to fill the chip: 4 wavefronts; the largest stream best with 8
    int waves = N * K >= (int64_t{1} << 27) ? 8 : 4;
    while (waves < passes) waves *= 2;
    if (waves > 8) return false;
    const int groups = waves / passes;
    const dim3 grid(static_cast<unsigned>((N + groups * kI8RowChannels - 1) / (groups * kI8RowChannels)));
    const int n = static_cast<int>(N), k = static_cast<int>(K);
#define TPQ_I8ROW(R, WV) int8_row_kernel<R, WV, Epilogue><<<grid, WV * kWave, 0, s>>>(a, w, n, k, passes, groups, ep)
#define TPQ_I8ROW_W(R) do { if (waves == 4) TPQ_I8ROW(R, 4); else TPQ_I8ROW(R, 8); } while (0)
    switch (rows) {
        case 1: TPQ_I8ROW_W(1); break;
        case 2: TPQ_I8ROW_W(2); break;
        case 3: TPQ_I8ROW_W(3); break;
        default: TPQ_I8ROW_W(4); break;
    }
#undef TPQ_I8ROW_W
#undef TPQ_I8ROW
    return true;
}

inline bool int8_decode_ok(const void* a, const void* w, int64_t M, int64_t N, int64_t K) {
    return M >= 1 && K >= 128 && K % 128 == 0 && aligned(a, 16) && aligned(w, 16) && N <= 0x7FFFFFF0 && K <= 0x7FFFFF80;
}

inline int i8_flight_compute_units() {
    static std::atomic<int> cached{0};
    int v = cached.load(std::memory_order_relaxed);
    if (v == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        v = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) ? prop.multiProcessorCount : 256;
        cached.store(v, std::memory_order_relaxed);
    }
    return v;
}

template <int NB, int MB, int SPW, int XR, class Epilogue>
int launch_int8_flight_as(const int8_t* x, const int8_t* w, int rows, int N, int K, const Epilogue& ep, hipStream_t s) {
    constexpr size_t bytes = i8_flight_lds_bytes<NB, MB, XR>();
    static_assert(bytes <= 160 * 1024, "LDS of one compute unit");
    static std::atomic<uint64_t> reserved{0};
    const auto kernel = int8_flight_kernel<NB, MB, SPW, XR, Epilogue>;
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), bytes, reserved, "int8 decode gemm (all in flight)")) return rc;
    kernel<<<dim3((N + 16 * NB - 1) / (16 * NB)), dim3(kFlightWaves * kWave), bytes, s>>>(x, w, rows, N, K, ep);
    return check_launch("int8 decode gemm (all in flight)");
}

// 3..32 rows on the all-in-flight kernel (int8_flight_kernel.h); false when the shape is not one of its cases
template <class Epilogue>
bool launch_int8_flight(const int8_t* x, const int8_t* w, int rows, int N, int K, const Epilogue& ep, hipStream_t s, int* rc) {
    const int steps = K / 128;
    const int spw = (steps + kFlightWaves - 1) / kFlightWaves;
    // Measured (us, bf16 out, loop kernel -> this one): 4096 x 4096 at 16 / 32 rows 7.2 / 9.9 -> 6.2 / 7.1; 4096 -> 11008 at 8 / 16 / 32
    // rows 13.4 / 15.5 / 20.9 -> 11.4 / 11.9 / 18.0; 4096 -> 32000 at 16 rows 34.0 -> 29.0; 8192 x 8192 at 16 rows 18.3 -> 16.7.
    // Not with one step per wavefront (2048 -> 4096 at 8 rows: 5.1 us against 4.7) and not beyond 16 rows at long K (even).
    if (steps < 2 * kFlightWaves - 8 || spw > 4 || rows > 32 || (spw > 2 && rows > 16)) return false;
    const int blocks = (N + 15) / 16, cus = i8_flight_compute_units();
    const int widest = spw <= 2 ? (rows > 16 ? 2 : 4) : 2;
    int nb = 0;
    for (int c = 1; c <= widest && nb == 0; ++c)
        if ((blocks + c - 1) / c <= cus) nb = c;
    if (nb == 0 && spw <= 2) nb = widest;
    if (const char* env = tuning_env("TPQ_INT8_FLIGHT")) nb = std::atoi(env);  // 0 switches the kernel off, 1..4 pin the width
    if (nb <= 0 || nb > widest) return false;
#define TPQ_I8F(NBV, MBV, SPWV, XRV) *rc = launch_int8_flight_as<NBV, MBV, SPWV, XRV, Epilogue>(x, w, rows, N, K, ep, s)
#define TPQ_I8F_ROWS(NBV, SPWV) do { if (rows <= 8) TPQ_I8F(NBV, 1, SPWV, 8); else TPQ_I8F(NBV, 1, SPWV, 16); } while (0)
    if (rows > 16) { if (nb == 1) TPQ_I8F(1, 2, 2, 32); else TPQ_I8F(2, 2, 2, 32); }
    else if (spw <= 2) { if (nb == 1) TPQ_I8F_ROWS(1, 2); else if (nb == 2) TPQ_I8F_ROWS(2, 2); else if (nb == 3) TPQ_I8F_ROWS(3, 2); else TPQ_I8F_ROWS(4, 2); }
    else if (spw == 3) { if (nb == 1) TPQ_I8F_ROWS(1, 3); else TPQ_I8F_ROWS(2, 3); }
    else { if (nb == 1) TPQ_I8F_ROWS(1, 4); else TPQ_I8F_ROWS(2, 4); }
#undef TPQ_I8F_ROWS
#undef TPQ_I8F
    return true;
}

// slabs of 32 rows (16 for what is left); the epilogue sees row indices of the whole problem through `rebase`
template <class Epilogue, class Rebase>
int launch_int8_decode(const int8_t* a, const int8_t* w, int64_t M, int64_t N, int64_t K, Epilogue ep, Rebase rebase, hipStream_t s) {
    static const int forced_nb = [] { const char* e = tuning_env("TPQ_INT8_DECODE_NB"); return e ? std::atoi(e) : 0; }();
    static const int forced_mb = [] { const char* e = tuning_env("TPQ_INT8_DECODE_MB"); return e ? std::atoi(e) : 0; }();
    static const int forced_waves = [] { const char* e = tuning_env("TPQ_INT8_DECODE_WAVES"); return e ? std::atoi(e) : 0; }();
    // One or two rows: the row kernel.  Measured against the matrix-core kernel below (us, one row): 4096 x 4096 5.3 / 5.6,
    // 11008 -> 4096 9.8 / 13.6, 4096 -> 11008 10.0 / 12.6, 8192 x 8192 13.5 / 16.2, 8192 -> 28672 38.1 / 46.2, 28672 -> 8192
    // 36.9 / 51.2 (6.4 TB/s); two rows: 10.5 / 13.4, 10.4 / 11.4, 14.5 / 16.3, 38.8 / 47.1, 38.3 / 52.6.  At four rows
    // the two are even (4096 x 4096: 6.8 / 5.9; 8192 x 8192: 15.8 / 17.4; 8192 -> 28672: 53.6 / 50.5) and the matrix-core
    // kernel stays.  A test-hook build pins it: never / up to four rows (route_override_int8_row).
    const int row_override = route_override_int8_row();
    const int row_limit = row_override < 0 ? 2 : row_override == 0 ? 0 : 4;
    if (M <= row_limit && launch_int8_rows(a, w, static_cast<int>(M), N, K, ep, s)) return check_launch("int8 row gemm");
    const int steps = static_cast<int>(K / 128);
    const int n = static_cast<int>(N), k = static_cast<int>(K);
    for (int64_t m0 = 0; m0 < M;) {
        const int left = static_cast<int>(M - m0 < 32 ? M - m0 : 32);
        {
            int rc = TPQ_OK;
            if (launch_int8_flight(a + m0 * K, w, left, static_cast<int>(N), static_cast<int>(K), rebase(ep, m0), s, &rc)) {
                if (rc != TPQ_OK) return rc;
                m0 += left;
                continue;
            }
        }
        const int mb = forced_mb ? forced_mb : (left > 16 ? 2 : 1);
        const int rows = left < 16 * mb ? left : 16 * mb;
        // Workgroup shape from a sweep over model shapes (K, N = 1024..28672): 32 channels pay from 8 rows on where
        // N gives a whole number of rounds of workgroups (8192 x 8192, 32 rows: 22.4 us against 26.3; 28672 -> 8192:
        // 69 against 86), never for one row or narrow N (4096 x 4096, 16 rows: 9.3 us against 6.9).
        const bool wide = rows >= 8 && ((N >= 6144 && N < 10240) || N >= 16384);
        const int nb = forced_nb ? forced_nb : (wide ? 2 : 1);
        const int waves = forced_waves ? forced_waves : (nb == 2 ? 8 : mb == 2 ? 4 : steps >= 32 ? 8 : 4);
        const dim3 grid(static_cast<unsigned>((N + 16 * nb - 1) / (16 * nb)));
        const Epilogue slab = rebase(ep, m0);
        const int8_t* xs = a + m0 * K;
#define TPQ_I8DEC(NBV, MBV, WV) int8_decode_kernel<NBV, MBV, WV, Epilogue><<<grid, WV * kWave, 0, s>>>(xs, w, rows, n, k, slab)
        if (nb == 2 && mb == 2) { if (waves == 8) TPQ_I8DEC(2, 2, 8); else TPQ_I8DEC(2, 2, 4); }
        else if (nb == 2) { if (waves == 8) TPQ_I8DEC(2, 1, 8); else TPQ_I8DEC(2, 1, 4); }
        else if (mb == 2) { if (waves == 8) TPQ_I8DEC(1, 2, 8); else TPQ_I8DEC(1, 2, 4); }
        else { if (waves == 8) TPQ_I8DEC(1, 1, 8); else TPQ_I8DEC(1, 1, 4); }
#undef TPQ_I8DEC
        m0 += rows;
    }
    return check_launch("int8 decode gemm");
}

}  // namespace
}  // namespace tpq
