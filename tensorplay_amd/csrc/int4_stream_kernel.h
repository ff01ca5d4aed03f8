// Streaming int4 decode kernel (one activation row): contiguous reads, every
// compute unit busy.
//
// The 128-byte unit of the packed layout is (tile nT, k-tile kT): 8 rows x 16
// bytes, and consecutive k-tiles of one tile are adjacent in memory.  A
// wavefront owns one tile and one half of the k range and reads it 1 KB at a
// time: lane l takes the 16 bytes of row l%8 in k-tile kt0 + l/8, so the 64
// lanes cover 8 consecutive k-tiles = 1024 contiguous bytes per load, eight
// such loads in flight.  A workgroup owns T consecutive tiles (2T wavefronts)
// with T = ceil(tiles / compute units): the tiles are dealt evenly over the
// whole chip and no reduction leaves the workgroup.
//
// The eight lane groups of a wavefront work on different k-tiles, so the
// activations come from LDS: the workgroup stages x once (20-word stride per
// k-tile, so that the eight groups' 16-byte reads fall in distinct banks while
// the lanes of a group read one address) next to two numbers per k-tile for
// the offset correction, and every lane fetches the 16 words of its k-tile
// with four ds_read_b128, one load ahead of the arithmetic.  The activation
// loads are issued BEFORE the weight loads: vector loads of a wavefront retire
// in order, so the staging barrier only waits for x and the weights are
// consumed load by load as they arrive.
//
// Arithmetic per lane and load (32 k of one row): 4 shifts + 16 v_and_or_b32
// turn the nibbles into fp16 pairs (magic + c); eight v_mfma_f32_4x4x4_16B_f16
// multiply them with the activations.  The four lanes of a 4x4x4 block share
// their k-tile, hence their activations: with A = activations and B = the
// lane's weights every accumulator register of the lane holds the lane's own
// dot product p = sum x (magic + c).  It is folded at once in fp32:
//   y += scale * (p - corr) + zero * sx,   corr = sum x (magic + 8), sx = sum x
// (corr and sx per k-tile come from the staging pass).  bf16 activations use
// v_dot2_f32_bf16 instead of the matrix instruction.  Lane groups are added
// with three butterfly steps, the two halves of the k range in LDS.
#pragma once

#include "int4_lane.h"

namespace tpq {
namespace {

constexpr int kXStride = 20;     // LDS words per k-tile of activations (16 used)
constexpr int kStreamLoads = 8;  // 1 KB loads in flight per wavefront

// EXACT: both halves of the k range are whole multiples of 8 k-tiles (k_super % 16 == 0), so no
// lane ever runs past its half and the per-load index clamps disappear.
template <int DT, int GROUP_KT, bool EXACT>
__global__ __launch_bounds__(1024) void int4_stream_kernel(
    const uint32_t* __restrict__ x, const uint4* __restrict__ packed, const uint32_t* __restrict__ sz,
    uint16_t* __restrict__ y, int N, int k_super, int n_tiles, int tiles_per_block) {
    using L = Lane16<DT>;
    extern __shared__ uint32_t lds[];
    uint32_t* xl = lds;                                                // [k_super][kXStride]
    float2* xs = reinterpret_cast<float2*>(lds + k_super * kXStride);  // [k_super] (corr, sx)
    float* red = reinterpret_cast<float*>(xs + k_super);               // [waves][8]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 3, r = lane & 7;
    const int tile = blockIdx.x * tiles_per_block + (wave >> 1);
    const bool live = tile < n_tiles;                                  // wave-uniform
    const int k_half = ((k_super + 15) / 16) * 8;                      // first half: multiple of 8 k-tiles
    const int kt_begin = (wave & 1) ? k_half : 0;
    const int kt_end = (wave & 1) ? k_super : (k_half < k_super ? k_half : k_super);

    // ---- activations first: 16 bytes per thread (word group w4 of k-tile kt) ------------------
    const int x_chunks = k_super * 4;
    uint4 xv0 = make_uint4(0, 0, 0, 0);
    if (tid < x_chunks) xv0 = reinterpret_cast<const uint4*>(x)[tid];

    // ---- then the first batch of weights --------------------------------------------------------
    const int kt_lane = kt_begin + g;
    const uint4* wl = packed + (static_cast<size_t>(live ? tile : 0) * k_super + kt_lane) * 8 + r;
    const uint32_t* szl = sz + static_cast<size_t>(kt_lane / GROUP_KT) * N + (live ? tile * 8 + r : 0);
    const size_t sz_step = static_cast<size_t>(8 / GROUP_KT) * N;      // eight k-tiles further
    const uint32_t* xl_lane = xl + kt_lane * kXStride;
    const float2* xs_lane = xs + kt_lane;

    uint4 q[kStreamLoads];
    uint32_t p[kStreamLoads];
    auto issue = [&](int batch_kt) {  // batch_kt: first k-tile of the batch (wave-uniform)
#pragma unroll
        for (int u = 0; u < kStreamLoads; ++u) {
            if constexpr (EXACT) {
                q[u] = wl[u * 64];
                p[u] = szl[u * sz_step];
            } else {  // past the end of the half: re-read the last k-tile, the result is dropped
                const int over = batch_kt + u * 8 + g - (kt_end - 1);
                const int back = over > 0 ? over : 0;
                q[u] = wl[u * 64 - back * 8];
                p[u] = sz[static_cast<size_t>((batch_kt + u * 8 + g - back) / GROUP_KT) * N + (live ? tile * 8 + r : 0)];
            }
        }
    };
    if (live && kt_begin < kt_end) issue(kt_begin);

    // ---- stage x and the two correction terms per k-tile --------------------------------------
    // thread t holds words 4j..4j+3 (pair index j = t%4) of k-tile t/4; even and odd j use
    // different magic exponents, so their sums are kept apart until the correction is formed
    for (int c = tid; c < x_chunks; c += blockDim.x) {
        const uint4 v = c == tid ? xv0 : reinterpret_cast<const uint4*>(x)[c];
        const int kt = c >> 2, j = c & 3;
        *reinterpret_cast<uint4*>(xl + kt * kXStride + 4 * j) = v;
        float s = L::dot(v.x, L::kOnes, 0.0f);
        s = L::dot(v.y, L::kOnes, s);
        s = L::dot(v.z, L::kOnes, s);
        s = L::dot(v.w, L::kOnes, s);
        const float same = s + __shfl_xor(s, 2, kWave);          // j and j^2: same parity
        const float other = __shfl_xor(same, 1, kWave);          // the other parity
        if (j == 0) xs[kt] = make_float2(__builtin_fmaf(L::kOffsetEven, same, L::kOffsetOdd * other), same + other);
    }
    __syncthreads();

    uint32_t magic_even, magic_odd;  // kept in VGPRs: v_and_or_b32 takes one scalar operand only
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_even) : "s"(L::kMagicEven));
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic_odd) : "s"(L::kMagicOdd));

    float yacc = 0.0f;
    if (live) {
        for (int batch = kt_begin; batch < kt_end; batch += kStreamLoads * 8) {
            const int off_x = (batch - kt_begin) * kXStride, off_s = batch - kt_begin;
            auto x_of = [&](int u, uint4 (&xr)[4], float2& sx, int& back) {
                back = 0;
                if constexpr (!EXACT) {
                    const int over = batch + u * 8 + g - (kt_end - 1);
                    back = over > 0 ? over : 0;
                }
                const uint4* xv = reinterpret_cast<const uint4*>(xl_lane + off_x + (u * 8 - back) * kXStride);
                xr[0] = xv[0]; xr[1] = xv[1]; xr[2] = xv[2]; xr[3] = xv[3];
                sx = xs_lane[off_s + u * 8 - back];
            };
            uint4 xn[4];
            float2 sxn;
            int backn;
            x_of(0, xn, sxn, backn);
#pragma unroll
            for (int u = 0; u < kStreamLoads; ++u) {
                if (batch + u * 8 < kt_end) {  // wave-uniform
                    const uint4 x0 = xn[0], x1 = xn[1], x2 = xn[2], x3 = xn[3];
                    const float2 sx = sxn;
                    const int back = backn;
                    if (u + 1 < kStreamLoads && batch + (u + 1) * 8 < kt_end) x_of(u + 1, xn, sxn, backn);
                    const uint32_t xw[16] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w,
                                             x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
                    const uint32_t wq[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
                    uint32_t v[4][4];
#pragma unroll
                    for (int t4 = 0; t4 < 4; ++t4) L::template unpack<L::kUseMfma>(wq[t4], v[t4], magic_even, magic_odd);
                    float part;
                    if constexpr (L::kUseMfma) {
                        float4_t acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                        for (int j = 0; j < 4; ++j) {  // word t4 + 4j of x pairs with pair j of word t4
                            acc0 = L::mfma(xw[4 * j], xw[4 * j + 1], v[0][j], v[1][j], acc0);
                            acc1 = L::mfma(xw[4 * j + 2], xw[4 * j + 3], v[2][j], v[3][j], acc1);
                        }
                        part = acc0[0] + acc1[0];
                    } else {
                        part = 0.0f;
#pragma unroll
                        for (int j = 0; j < 4; ++j)
#pragma unroll
                            for (int t4 = 0; t4 < 4; ++t4) part = L::dot(xw[t4 + 4 * j], v[t4][j], part);
                    }
                    const float scale = L::lo(p[u]), zero = L::hi(p[u]);
                    const float contrib = __builtin_fmaf(zero, sx.y, scale * (part - sx.x));
                    if constexpr (EXACT) yacc += contrib;
                    else yacc += back == 0 ? contrib : 0.0f;
                }
            }
            if (batch + kStreamLoads * 8 < kt_end) {
                wl += kStreamLoads * 64;
                szl += kStreamLoads * sz_step;
                issue(batch + kStreamLoads * 8);
            }
        }
    }
    yacc += __shfl_xor(yacc, 8, kWave);
    yacc += __shfl_xor(yacc, 16, kWave);
    yacc += __shfl_xor(yacc, 32, kWave);
    if (lane < 8) red[wave * 8 + lane] = yacc;
    __syncthreads();
    if (tid < tiles_per_block * 8) {
        const int tl = tid >> 3, rr = tid & 7;
        const int nn = (blockIdx.x * tiles_per_block + tl) * 8 + rr;
        if (nn < N) y[nn] = L::out(red[(2 * tl) * 8 + rr] + red[(2 * tl + 1) * 8 + rr]);
    }
}

}  // namespace
}  // namespace tpq
