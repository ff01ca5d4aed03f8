// Launcher of the all-in-flight matrix-core int4 kernel: picks the workgroup width and the instantiation.
#include "int4_flight.h"

#include <cstdlib>

#include "int4_mfma_flight_kernel.h"
#include "int8pack_flight_kernel.h"

namespace tpq {
namespace {

inline int flight_compute_units() {
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

template <int DT, int NB, int SPW, int XR, int MODE, bool NORM, int RB = 1>
int launch_as(const uint16_t* x, int rows, const FlightSet& set, int blocks, int K, int shift, const uint16_t* residual, hipStream_t s) {
    constexpr size_t bytes = flight_lds_bytes<NB, SPW, XR>();
    static_assert(bytes <= 160 * 1024, "LDS of one compute unit");
    static std::atomic<uint64_t> reserved{0};
    const auto kernel = int4_mfma_flight_kernel<DT, NB, SPW, XR, MODE, NORM, RB>;
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), bytes, reserved, "tpq_int4_mm (mfma, all in flight)")) return rc;
    constexpr int C = MODE == kFlightPair ? NB / 2 : NB;
    kernel<<<dim3((blocks + C - 1) / C), dim3(kFlightWaves * kWave), bytes, s>>>(x, set, rows, K, shift, residual);
    return check_launch("tpq_int4_mm (mfma, all in flight)");
}

// the row capacity: 4, 8 or 16 rows through LDS
template <int DT, int NB, int SPW, int MODE>
int launch_rows(const uint16_t* x, int rows, const FlightSet& set, int blocks, int K, int shift, const uint16_t* residual, hipStream_t s) {
    if constexpr (SPW <= 4 && MODE != kFlightOne) {  // the normalizing form: built for K = 2048..8192, pair and several weights
        if (set.norm_weight != nullptr) {
            if (rows <= 4) return launch_as<DT, NB, SPW, 4, MODE, true>(x, rows, set, blocks, K, shift, residual, s);
            if (rows <= 8) return launch_as<DT, NB, SPW, 8, MODE, true>(x, rows, set, blocks, K, shift, residual, s);
            if constexpr (flight_lds_bytes<NB, SPW, 16>() <= 160 * 1024) {
                return launch_as<DT, NB, SPW, 16, MODE, true>(x, rows, set, blocks, K, shift, residual, s);
            } else {
                return TPQ_ERR_UNSUPPORTED;
            }
        }
    } else {
        if (set.norm_weight != nullptr) return TPQ_ERR_UNSUPPORTED;  // not reached: launch() excludes the case
    }
    if (rows <= 4) return launch_as<DT, NB, SPW, 4, MODE, false>(x, rows, set, blocks, K, shift, residual, s);
    if (rows <= 8) return launch_as<DT, NB, SPW, 8, MODE, false>(x, rows, set, blocks, K, shift, residual, s);
    if constexpr (flight_lds_bytes<NB, SPW, 16>() <= 160 * 1024 && SPW <= 4) {
        return launch_as<DT, NB, SPW, 16, MODE, false>(x, rows, set, blocks, K, shift, residual, s);
    } else {
        return TPQ_ERR_UNSUPPORTED;  // not reached: flight_shape() excludes the case
    }
}

// Workgroup width (blocks of 16 channels) for `blocks` blocks in all, or 0 when the kernel is not built for the case.
// spw = steps per wavefront; the registers hold spw x width weight loads in flight, so long K means narrow workgroups.
// Measured at K = 4096, fp16 (us, loop kernel / this kernel at widths 1, 2, 3, 4):
//   N = 4096, 8 rows: 5.4 / 4.5 5.1 5.6 6.3     N = 8192, 8 rows: 6.4 / 7.6 5.7 6.1 6.9
//   N = 11008, 8 rows: 8.4 / 10.5 9.2 6.7 7.4    N = 16384, 8 rows: 9.7 / 14.0 10.2 11.6 9.1
//   N = 32000, 2 rows: 17.0 / 17.4 14.5 16.9 14.9;  8 rows: 17.9 / 25.8 18.1 17.0 15.4
// One workgroup per compute unit and pass: the narrowest width that needs one pass.  Several passes pay off only with
// two steps per wavefront or at most four rows (5120 -> 13824, 8 rows: 11.7 us against 10.5 for the loop kernel;
// 8192 -> 10240: 16.2 against 13.2; at 2 rows 10.0 / 10.4 and 12.4 / 12.9): then the width with the fewest
// passes x width, or 2 for few rows (their small LDS tiles let two workgroups share a compute unit).
int flight_width(int blocks, int rows, int spw, bool pair, bool one_weight) {
    const int cus = flight_compute_units();
    const int widest = pair ? 3 : spw <= 2 ? 4 : spw <= 4 ? 2 : 1;
    // gate / up at one or two rows: one block of each (4096 -> 11008: 11.8 / 12.1 us against 12.5 / 12.5 for three)
    if (pair && rows <= 2) return 1;
    // One row of one weight: only narrow workgroups in one pass; wider weights belong to the column-per-lane kernel
    // (4096 -> 4096: 3.9 us against 4.5; 4096 -> 6144: 5.0 / 5.5; 14336 -> 4096: 9.0 / 10.2; but 4096 -> 11008: 6.6 / 6.35).
    const bool narrow_only = rows == 1 && one_weight;
    for (int nb = 1; nb <= widest; ++nb)
        if ((blocks + nb - 1) / nb <= cus) return narrow_only && nb > 2 ? 0 : nb;
    if (narrow_only || (spw > 2 && rows > 4)) return 0;
    if (rows <= 4 && widest >= 2 && !pair) return 2;
    int best = widest, cost = 1 << 30;
    for (int nb = widest; nb >= 1; --nb) {
        const int c = ((blocks + nb - 1) / nb + cus - 1) / cus * nb;
        if (c < cost) { cost = c; best = nb; }
    }
    return best;
}

template <int DT>
bool launch(const void* x, int rows, const FlightWeights& wts, int K, int group, bool pair, const void* residual, hipStream_t s, int* rc) {
    const bool norm = wts.norm_weight != nullptr;
    if (norm && (!aligned(wts.norm_weight, 16) || K > 8192)) return false;  // built for up to four steps per wavefront
    if (rows < 1 || rows > 32 || K % 128 != 0 || (group != 128 && group != 256) || !aligned(x, 16)) return false;
    const int steps = K / 128;
    const int spw = (steps + kFlightWaves - 1) / kFlightWaves;
    if (steps < kFlightWaves || spw > 7 || spw == 5) return false;
    // 17..32 rows: two blocks of 16 rows against the same weight registers; one weight, up to two steps per wavefront
    const bool two_blocks = rows > 16;
    if (two_blocks && (spw > 3 || pair || norm || tuning_env("TPQ_INT4_NO_TWO_BLOCKS"))) return false;
    // five and more steps per wavefront at more than eight rows: the tiles of 16 rows keep one step in LDS at a time and
    // the registers fill up (11008 -> 4096 at 16 rows: 17.7 us against 14.0 for the loop kernel)
    if (spw > 4 && rows > 8) return false;
    if (wts.count < 1 || wts.count > kFlightMaxWeights || (pair && (wts.count != 2 || wts.N[0] != wts.N[1] || spw != 2))) return false;
    // gate / up at more than eight rows: the tiles of 16 rows leave LDS for two blocks of each weight only, and the
    // loop kernel is faster then (4096 -> 11008 at 12 rows: 15.9 us against 17.1)
    if (pair && rows > 8) return false;
    if (residual != nullptr && (wts.count != 1 || pair || !aligned(residual, 8))) return false;
    FlightSet set{};
    FlightWeight* const slots[kFlightMaxWeights] = {&set.w0, &set.w1, &set.w2, &set.w3};
    set.count = pair ? 1 : wts.count;
    set.norm_weight = static_cast<const uint16_t*>(wts.norm_weight);
    set.norm_eps = wts.norm_eps;
    set.norm_inv_k = 1.0f / static_cast<float>(K);
    int blocks = 0;
    for (int w = 0; w < wts.count; ++w) {
        if (wts.N[w] % 8 != 0 || !aligned(wts.sz[w], 4) || !aligned(wts.packed[w], 16) || !aligned(wts.y[pair ? 0 : w], 8)) return false;
        slots[w]->packed = static_cast<const uint4*>(wts.packed[w]);
        slots[w]->sz = static_cast<const uint32_t*>(wts.sz[w]);
        slots[w]->y = static_cast<uint16_t*>(wts.y[pair ? 0 : w]);
        slots[w]->N = wts.N[w];
        slots[w]->first = pair ? 0 : blocks;
        if (!pair || w == 0) blocks += (wts.N[w] + 15) / 16;
    }
    int nb = flight_width(blocks, rows < 16 ? rows : 16, spw, pair, wts.count == 1);
    if (const char* env = tuning_env("TPQ_INT4_FLIGHT")) nb = std::atoi(env);  // 0 switches the kernel off, 1..4 pin the width
    if (nb <= 0) return false;
    // Two blocks of rows: measured against the loop kernel with two row blocks per workgroup (us, 17 / 24 / 32 rows):
    // 4096 -> 11008 11.5 / 11.4 / 11.3 against 11.4 / 11.9 / 13.2; 4096 x 4096 7.5 / 7.6 / 7.7 against 8.1 / 9.1 / 10.4;
    // 3072 -> 9216 9.3 / 9.2 / 9.5 against 13.1 / 15.1 / 17.5; 4096 -> 6144 8.6 / 8.7 / 8.9 against 8.8 / 9.8 / 11.3.  It loses
    // where the workgroups need more than one pass or the widest form (4096 -> 16384: 17.8 against 13.5 at 32 rows;
    // 4096 -> 32000: 32.5 against 25.5) and with a single step per wavefront (2048 -> 8192: 7.2 against 6.1 at 17 rows).
    // Three steps per wavefront (K up to 6144): only the form of one block per workgroup keeps everything in registers
    // (5120 -> 2560 at 17 / 24 / 32 rows: 8.7 / 8.9 / 9.3 against 9.4 / 10.7 / 12.5); two blocks per workgroup spill 17
    // registers and four steps 18..52, and lose by up to 2 x (8192 x 8192 at 32 rows: 34.9 against 19.4).
    if (two_blocks && (nb > 3 || (blocks + nb - 1) / nb > flight_compute_units() || steps < 24 || (spw == 3 && nb != 1))) return false;
    const auto* xp = static_cast<const uint16_t*>(x);
    const auto* rp = static_cast<const uint16_t*>(residual);
    const int shift = group == 128 ? 0 : 1;
    int code = TPQ_ERR_UNSUPPORTED;
    if (pair) {
        if (nb >= 3 && rows <= 8) code = launch_rows<DT, 6, 2, kFlightPair>(xp, rows, set, blocks, K, shift, rp, s);
        else if (nb >= 2) code = launch_rows<DT, 4, 2, kFlightPair>(xp, rows, set, blocks, K, shift, rp, s);
        else code = launch_rows<DT, 2, 2, kFlightPair>(xp, rows, set, blocks, K, shift, rp, s);
    } else {
#define TPQ_FLIGHT(NBV, SPWV)                                                                                   \
    code = wts.count == 1 && !norm ? launch_rows<DT, NBV, SPWV, kFlightOne>(xp, rows, set, blocks, K, shift, rp, s)    \
                          : launch_rows<DT, NBV, SPWV, kFlightMany>(xp, rows, set, blocks, K, shift, rp, s)
        switch (spw) {
            case 1: case 2:
                if (two_blocks) {
#define TPQ_FLIGHT2(NBV)                                                                                                   \
    code = wts.count == 1 ? launch_as<DT, NBV, 2, 16, kFlightOne, false, 2>(xp, rows, set, blocks, K, shift, rp, s)          \
                          : launch_as<DT, NBV, 2, 16, kFlightMany, false, 2>(xp, rows, set, blocks, K, shift, rp, s)
                    if (nb == 1) TPQ_FLIGHT2(1); else if (nb == 2) TPQ_FLIGHT2(2); else if (nb == 3) TPQ_FLIGHT2(3); else TPQ_FLIGHT2(4);
#undef TPQ_FLIGHT2
                    break;
                }
                if (nb == 1) TPQ_FLIGHT(1, 2); else if (nb == 2) TPQ_FLIGHT(2, 2); else if (nb == 3) TPQ_FLIGHT(3, 2); else TPQ_FLIGHT(4, 2);
                break;
            case 3:
                if (two_blocks) {  // one block per workgroup only (nb == 1: see above)
                    code = wts.count == 1 ? launch_as<DT, 1, 3, 16, kFlightOne, false, 2>(xp, rows, set, blocks, K, shift, rp, s)
                                          : launch_as<DT, 1, 3, 16, kFlightMany, false, 2>(xp, rows, set, blocks, K, shift, rp, s);
                    break;
                }
                if (nb == 1) TPQ_FLIGHT(1, 3); else TPQ_FLIGHT(2, 3);
                break;
            case 4: if (nb == 1) TPQ_FLIGHT(1, 4); else TPQ_FLIGHT(2, 4); break;
            case 6: TPQ_FLIGHT(1, 6); break;
            case 7: TPQ_FLIGHT(1, 7); break;
            default: return false;
        }
#undef TPQ_FLIGHT
    }
    *rc = code;
    return true;
}

template <int DT, int NB, int SPW, int XR, int RB = 1>
int launch_int8_as(const uint16_t* x, int rows, const int8_t* w, const float* scales, uint16_t* y, int N, int K, hipStream_t s) {
    constexpr size_t bytes = int8_flight_lds_bytes<NB, SPW, XR>();
    static_assert(bytes <= 160 * 1024, "LDS of one compute unit");
    static std::atomic<uint64_t> reserved{0};
    const auto kernel = int8pack_flight_kernel<DT, NB, SPW, XR, RB>;
    if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), bytes, reserved, "_weight_int8pack_mm (all in flight)")) return rc;
    kernel<<<dim3((N + 16 * NB - 1) / (16 * NB)), dim3(kFlightWaves * kWave), bytes, s>>>(x, w, scales, y, rows, N, K);
    return check_launch("_weight_int8pack_mm (all in flight)");
}

template <int DT, int NB, int SPW>
int launch_int8_rows(const uint16_t* x, int rows, const int8_t* w, const float* scales, uint16_t* y, int N, int K, hipStream_t s) {
    if (rows <= 4) return launch_int8_as<DT, NB, SPW, 4>(x, rows, w, scales, y, N, K, s);
    if (rows <= 8) return launch_int8_as<DT, NB, SPW, 8>(x, rows, w, scales, y, N, K, s);
    if constexpr (SPW <= 2) {
        if (rows > 16) return launch_int8_as<DT, NB, SPW, 16, 2>(x, rows, w, scales, y, N, K, s);  // two blocks of 16 rows
        return launch_int8_as<DT, NB, SPW, 16>(x, rows, w, scales, y, N, K, s);
    } else {
        return TPQ_ERR_UNSUPPORTED;  // not reached
    }
}

// Measured (fp16, us, loop kernel -> this one): 4096 -> 11008 at 3 / 8 / 16 rows 14.4 / 16.6 / 20.7 -> 11.5 / 12.1 / 13.1;
// 4096 x 4096 at 8 rows 7.5 -> 6.4; 4096 -> 32000 at 8 rows 34.7 -> 28.5; 11008 -> 4096 at 8 rows 16.2 -> 14.2.
template <int DT>
bool launch_int8(const void* x, int rows, const int8_t* w, const float* scales, void* y, int N, int K, hipStream_t s, int* rc) {
    if (rows < 1 || rows > 32 || K % 128 != 0 || !aligned(x, 16) || !aligned(w, 16)) return false;
    const int steps = K / 128;
    const int spw = (steps + kFlightWaves - 1) / kFlightWaves;
    // 17..32 rows: two blocks of 16 rows against the same weight registers, up to two steps per wavefront, one pass of workgroups
    const bool two_blocks = rows > 16;
    if (two_blocks && (spw > 2 || steps < 24 || tuning_env("TPQ_INT8PACK_NO_TWO_BLOCKS"))) return false;
    // more than two steps per wavefront at more than eight rows: the loop kernel is as fast or faster (8192 x 8192 at 12 rows:
    // 22.0 us against 19.5; 11008 -> 4096: 17.8 / 17.8)
    if (steps < kFlightWaves || spw > 7 || spw == 5 || (spw > 2 && rows > 8)) return false;
    const int blocks = (N + 15) / 16;
    const int cus = flight_compute_units();
    const int widest = spw <= 2 ? 4 : spw <= 4 ? 2 : 1;
    int nb = 0;
    for (int c = 1; c <= widest && nb == 0; ++c)
        if ((blocks + c - 1) / c <= cus) nb = c;
    if (nb == 0 && spw <= 2) nb = widest;  // several passes pay off with two steps per wavefront only (see flight_width)
    if (const char* env = tuning_env("TPQ_INT8PACK_FLIGHT")) nb = std::atoi(env);  // 0 switches the kernel off, 1..4 pin the width
    if (nb <= 0 || nb > widest) return false;
    // Two blocks of rows, measured against the loop kernel with two row blocks per workgroup (us, 17 / 24 / 32 rows):
    // 4096 -> 11008 15.2 / 15.4 / 15.8 against 24.3 / 28.1 / 32.0; 4096 x 4096 8.7 / 9.2 / 9.6 against 10.4 / 11.9 / 13.3;
    // 3072 -> 9216 14.2 / 14.6 / 15.0 against 20.1 / 21.9 / 23.9; the widest form loses (4096 -> 16384: 34.0 against 31.1)
    if (two_blocks && (nb > 3 || (blocks + nb - 1) / nb > cus)) return false;
    const auto* xp = static_cast<const uint16_t*>(x);
    auto* yp = static_cast<uint16_t*>(y);
    int code = TPQ_ERR_UNSUPPORTED;
#define TPQ_FLIGHT8(NBV, SPWV) code = launch_int8_rows<DT, NBV, SPWV>(xp, rows, w, scales, yp, N, K, s)
    switch (spw) {
        case 1: case 2:
            if (nb == 1) TPQ_FLIGHT8(1, 2); else if (nb == 2) TPQ_FLIGHT8(2, 2); else if (nb == 3) TPQ_FLIGHT8(3, 2); else TPQ_FLIGHT8(4, 2);
            break;
        case 3: if (nb == 1) TPQ_FLIGHT8(1, 3); else TPQ_FLIGHT8(2, 3); break;
        case 4: if (nb == 1) TPQ_FLIGHT8(1, 4); else TPQ_FLIGHT8(2, 4); break;
        case 6: TPQ_FLIGHT8(1, 6); break;
        case 7: TPQ_FLIGHT8(1, 7); break;
        default: return false;
    }
#undef TPQ_FLIGHT8
    *rc = code;
    return true;
}

}  // namespace

bool flight_launch_int8pack(int dtype, const void* x, int rows, const int8_t* w, const float* scales, void* y, int N, int K,
                            hipStream_t stream, int* rc) {
    if (dtype == TPQ_DTYPE_F16) return launch_int8<TPQ_DTYPE_F16>(x, rows, w, scales, y, N, K, stream, rc);
    if (dtype == TPQ_DTYPE_BF16) return launch_int8<TPQ_DTYPE_BF16>(x, rows, w, scales, y, N, K, stream, rc);
    return false;
}

bool flight_launch(int dtype, const void* x, int rows, const FlightWeights& weights, int K, int group, bool pair,
                   const void* residual, hipStream_t stream, int* rc) {
    if (dtype == TPQ_DTYPE_F16) return launch<TPQ_DTYPE_F16>(x, rows, weights, K, group, pair, residual, stream, rc);
    if (dtype == TPQ_DTYPE_BF16) return launch<TPQ_DTYPE_BF16>(x, rows, weights, K, group, pair, residual, stream, rc);
    return false;
}

}  // namespace tpq
