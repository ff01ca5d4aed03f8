// Ternary-weight product for a few activation rows (1..16 MB per launch: decode batches of the BitNet
// linear), K % 256 == 0.  The packed weight is streamed once whatever the row count:
// v_mfma_i32_16x16x64_i8 with the WEIGHTS as the A operand, NB blocks of 16 channels per workgroup.
// Lane (i, q) owns weight row n0 + i and, in a step of 256 k, the 16 packed bytes (64 codes) at
// k = 256 s + 64 q: one 16-byte load, four MFMAs (one per packed dword).
//
// Expanding a packed dword w (bytes b = 0..3, the code of k = 4 b + j in bits 7-2j..6-2j of byte b) the
// cheap way gives the codes of ONE field position per register: (w >> (6 - 2 j)) & 0x03030303 holds
// the four codes k = j, 4 + j, 8 + j, 12 + j as bytes, and v_perm_b32 with those bytes as selectors
// into the table {0, 1, -2, -1} sign-extends them: 3 instructions per int8 dword.  Which k sits in
// which slot of the MFMA is free as long as both operands agree, so the activations are brought into
// the same order instead: lane (m, q) loads x[m][256 s + 64 q .. + 64) as four 16-byte chunks and
// transposes each as a 4 x 4 byte matrix (8 v_perm_b32), once for all NB channel blocks.
// D comes out as lane (m, q) x channels 4 q + v of a block in int32, exact; the wavefronts of a
// workgroup take the steps round-robin and add their partial sums through LDS.
//
// The activations of a step are 256 bytes = two cache lines per row.  Asked for in the MFMA's order (lane (m, q): 16
// bytes at 64 q + 16 d of row m, four loads) every load touches two lines of every row, 8 M line look-ups per step, and
// the vector memory path charges a load by the lines it touches: at 8 rows the activations cost it four times what the
// packed weights do.  So a wavefront reads them as they lie (lane l: 16 bytes at 16 (l % 16) of row l / 16, four rows =
// 8 whole lines per load, ceil(M / 4) loads), transposes what it got and passes it to the MFMA's lanes through a
// wave-private LDS area (row pitch 272 bytes, so the sixteen rows of a 16-byte read spread over the banks).  Columns
// m >= M hold whatever is there; their sums are dropped.
#pragma once

#include <cstdlib>

#include "int8_gemm_kernel.h"

namespace tpq {
namespace {

// 16 consecutive int8 (k0 .. k0 + 15) -> register j holds k0 + j, 4 + j, 8 + j, 12 + j
__device__ __forceinline__ v4i transpose_4x4_bytes(const uint4 r) {
    const uint32_t lo01 = __builtin_amdgcn_perm(r.y, r.x, 0x05010400u), hi01 = __builtin_amdgcn_perm(r.y, r.x, 0x07030602u);
    const uint32_t lo23 = __builtin_amdgcn_perm(r.w, r.z, 0x05010400u), hi23 = __builtin_amdgcn_perm(r.w, r.z, 0x07030602u);
    v4i out;
    out[0] = static_cast<int>(__builtin_amdgcn_perm(lo23, lo01, 0x05040100u));
    out[1] = static_cast<int>(__builtin_amdgcn_perm(lo23, lo01, 0x07060302u));
    out[2] = static_cast<int>(__builtin_amdgcn_perm(hi23, hi01, 0x05040100u));
    out[3] = static_cast<int>(__builtin_amdgcn_perm(hi23, hi01, 0x07060302u));
    return out;
}

// one packed dword (16 codes) -> register j holds the codes of field position j of its four bytes
__device__ __forceinline__ v4i ternary_fields_to_i8(uint32_t w) {
    constexpr uint32_t kTable = 0xFFFE0100u;  // selector 0..3 -> 0, 1, -2, -1
    v4i out;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        out[j] = static_cast<int>(__builtin_amdgcn_perm(0u, kTable, (w >> (6 - 2 * j)) & 0x03030303u));
    return out;
}

constexpr int kTdecXPitch = 272;                    // bytes per activation row in the exchange area
constexpr int kTdecXBytes = 16 * kTdecXPitch;      // per wavefront: 16 rows of one step

// XL: wave-level loads of activations per step (four rows each), rows <= 4 XL; MB = 2 takes XL = 8 (rows 16.. in the
// second block)
template <int NB, int MB, int XL, int WAVES, class Epilogue>
__global__ __launch_bounds__(WAVES * kWave) void ternary_decode_mfma_kernel(const int8_t* __restrict__ x, const uint8_t* __restrict__ packed,
                                                                           int m_base, int M, int N, int K, Epilogue ep) {
    static_assert(XL <= 4 * MB && (MB == 1 || XL == 8), "activation loads per step");
    __shared__ int red[WAVES][NB * MB][4][kWave];
    extern __shared__ __align__(16) unsigned char tdec_xch[];  // [WAVES][kTdecXBytes]
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int steps = K / 256;
    const int n0 = blockIdx.x * (16 * NB);
    const size_t bpr = static_cast<size_t>(K) >> 2;
    const uint4* w_base[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int n = n0 + 16 * b + i;
        w_base[b] = reinterpret_cast<const uint4*>(packed + static_cast<size_t>(n < N ? n : N - 1) * bpr) + q;  // rows past N: a valid row, result dropped
    }
    bool row_live[MB];
#pragma unroll
    for (int r = 0; r < MB; ++r) row_live[r] = 16 * r + i < M;
    // load j of a step: row 4 j + lane / 16, bytes 16 (lane % 16) of the step's 256 (rows past M: row 0, dropped)
    const uint4* x_base[XL];
#pragma unroll
    for (int j = 0; j < XL; ++j) {
        const int row = 4 * j + (lane >> 4);
        x_base[j] = reinterpret_cast<const uint4*>(x + static_cast<size_t>(m_base + (row < M ? row : 0)) * K) + (lane & 15);
    }
    unsigned char* const xch = tdec_xch + wave * kTdecXBytes;
    unsigned char* const xch_put = xch + (lane >> 4) * kTdecXPitch + (lane & 15) * 16;  // + 4 j rows
    const unsigned char* const xch_get = xch + i * kTdecXPitch + q * 64;                // + 16 d

    struct Step {
        uint4 w[NB];
        uint4 xv[XL];
    };
    auto load = [&](int s, Step& st) {
#pragma unroll
        for (int b = 0; b < NB; ++b) st.w[b] = nt_load(w_base[b] + s * 4);
#pragma unroll
        for (int j = 0; j < XL; ++j) st.xv[j] = x_base[j][s * 16];
    };
    v4i acc[NB][MB][2] = {};  // two accumulators per output block taking turns
    auto compute = [&](const Step& st) {
        v4i xb[MB][4];
#pragma unroll
        for (int r = 0; r < MB; ++r) {
            // this block's rows into the exchange area (LDS keeps a wavefront's accesses in order: the reads of the
            // block before are served before these writes), then each lane's four pieces out of it
#pragma unroll
            for (int j = 4 * r; j < 4 * r + 4 && j < XL; ++j) {
                const v4i f = transpose_4x4_bytes(st.xv[j]);
                *reinterpret_cast<v4i*>(xch_put + (j - 4 * r) * 4 * kTdecXPitch) = f;
            }
#pragma unroll
            for (int d = 0; d < 4; ++d) xb[r][d] = *reinterpret_cast<const v4i*>(xch_get + d * 16);
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint32_t word = d == 0 ? st.w[b].x : d == 1 ? st.w[b].y : d == 2 ? st.w[b].z : st.w[b].w;
                const v4i codes = ternary_fields_to_i8(word);
#pragma unroll
                for (int r = 0; r < MB; ++r) acc[b][r][d & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(codes, xb[r][d], acc[b][r][d & 1], 0, 0, 0);
            }
        }
    };

    // this wavefront's steps: wave, wave + WAVES, ...; RING in flight (a step is 16 (NB + XL) bytes per lane)
    constexpr int kRing = MB >= 2 ? 2 : 4;
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

    // The finishing wavefront asks for its row scales and bias values here, ahead of the exchange of the partial sums:
    // fetched element by element in the store loop each is a trip to memory that the next store waits for (a load
    // behind a store to `out` cannot be moved ahead of it).
    float row_scale[MB], bias_n[NB][4];
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < MB; ++r) row_scale[r] = ep.row_scale_of(m_base + (row_live[r] ? 16 * r + i : 0));
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int n = n0 + 16 * b + 4 * q + v;
                bias_n[b][v] = ep.bias_of(n < N ? n : N - 1);
            }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < MB; ++r)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][b * MB + r][v][lane] = acc[b][r][0][v] + acc[b][r][1][v];
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
                    const int n = n0 + 16 * b + 4 * q + v, m = m_base + 16 * r + i;
                    if (row_live[r] && n < N) ep.store_scaled(static_cast<int64_t>(m) * N + n, sum, row_scale[r], bias_n[b][v]);
                }
    }
}

inline bool ternary_decode_mfma_ok(const void* x, const void* packed, int64_t M, int64_t N, int64_t K) {
    return M >= 1 && N >= 1 && K >= 256 && K % 256 == 0 && aligned(x, 16) && aligned(packed, 16) && M <= 0x7FFFFFF0 && N <= 0x7FFFFFF0 &&
           K <= 0x7FFFFF00;
}

// slabs of 32 rows (16 for what is left)
template <class Epilogue>
int launch_ternary_decode_mfma(const int8_t* x, const uint8_t* packed, int64_t M, int64_t N, int64_t K, Epilogue ep, hipStream_t s) {
    static const int forced_nb = [] { const char* e = tuning_env("TPQ_TERNARY_NB"); return e ? std::atoi(e) : 0; }();
    static const int forced_mb = [] { const char* e = tuning_env("TPQ_TERNARY_MB"); return e ? std::atoi(e) : 0; }();
    static const int forced_waves = [] { const char* e = tuning_env("TPQ_TERNARY_WAVES"); return e ? std::atoi(e) : 0; }();
    // Workgroup shape from a sweep over model shapes (K 2560..28672, 1..16 rows), about 2000..4000 wavefronts in all:
    //   N < 8192: 16 channels x 8 wavefronts (4096 x 4096, 8 rows: 5.0 us; 32 channels: 6.6)
    //   N < 10240: 32 x 8 (8192 x 28672 -> 8192, 16 rows: 26.4 us; 16 channels: 36.3)
    //   N < 16384: 16 x 4 (4096 -> 11008, 2 rows: 6.7 us; 8 wavefronts 7.6, 32 channels 7.9)
    //   above: 32 x 4 (8192 -> 28672, 8 rows: 24.3 us; 16 channels 28.2, 8 wavefronts 29.4)
    const int nb = forced_nb ? forced_nb : ((N >= 8192 && N < 10240) || N >= 16384 ? 2 : 1);
    //   at most 256 workgroups of 16 channels and 24 steps of K or more: 16 wavefronts, two steps each instead of four
    //   (6912 -> 2560 at 8 rows 5.4 -> 5.1 us in the sweep's harness; 2560 -> 6912, 432 workgroups: 4.7 -> 6.5, stays at 8)
    const bool long_and_narrow = nb == 1 && N <= 16 * 256 && K >= 24 * 256;
    const int waves = forced_waves ? forced_waves : (long_and_narrow ? 16 : N < 10240 ? 8 : 4);
    const dim3 grid(static_cast<unsigned>((N + 16 * nb - 1) / (16 * nb)));
    const int n = static_cast<int>(N), k = static_cast<int>(K);
    for (int64_t m0 = 0; m0 < M;) {
        const int left = static_cast<int>(M - m0 < 32 ? M - m0 : 32);
        const int mb = forced_mb ? forced_mb : (left > 16 ? 2 : 1);
        const int rows = left < 16 * mb ? left : 16 * mb;
        const int base = static_cast<int>(m0);
        const int xl = rows > 16 ? 8 : rows > 8 ? 4 : rows > 4 ? 2 : 1;
        const size_t xch_bytes = static_cast<size_t>(waves) * kTdecXBytes;
#define TPQ_TDEC(NBV, MBV, XLV, WV)                                                                                      \
    do {                                                                                                                 \
        auto kernel = ternary_decode_mfma_kernel<NBV, MBV, XLV, WV, Epilogue>;                                           \
        constexpr size_t kStatic = sizeof(int) * WV * NBV * MBV * 4 * kWave;                                             \
        if (kStatic + xch_bytes > 64 * 1024) {                                                                           \
            static std::atomic<uint64_t> configured{0};                                                                  \
            if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), xch_bytes, configured, "tpq_ternary_mm (mfma decode)")) return rc; \
        }                                                                                                                \
        kernel<<<grid, WV * kWave, xch_bytes, s>>>(x, packed, base, rows, n, k, ep);                                     \
    } while (0)
#define TPQ_TDEC_X(NBV, WV)                                      \
    do {                                                         \
        if (mb == 2) TPQ_TDEC(NBV, 2, 8, WV);                    \
        else if (xl == 4) TPQ_TDEC(NBV, 1, 4, WV);               \
        else if (xl == 2) TPQ_TDEC(NBV, 1, 2, WV);               \
        else TPQ_TDEC(NBV, 1, 1, WV);                            \
    } while (0)
        if (nb == 2) { if (waves == 8) TPQ_TDEC_X(2, 8); else TPQ_TDEC_X(2, 4); }
        else { if (waves == 16) TPQ_TDEC_X(1, 16); else if (waves == 8) TPQ_TDEC_X(1, 8); else TPQ_TDEC_X(1, 4); }
#undef TPQ_TDEC_X
#undef TPQ_TDEC
        m0 += rows;
    }
    return check_launch("tpq_ternary_mm (mfma decode)");
}

}  // namespace
}  // namespace tpq
