// Internal helpers shared by the gfx950 kernels: error reporting, dtype
// conversion on the device, wavefront (64-lane) reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/tpq.h"

#define TPQ_EXPORT extern "C" __attribute__((visibility("default")))

namespace tpq {

constexpr int kWave = 64;

char* error_buffer();
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TPQ_ERR_RUNTIME, "%s: %s", what, hipGetErrorString(e));
    return TPQ_OK;
}

#define TPQ_REQUIRE(cond, code, ...)                    \
    do {                                                \
        if (!(cond)) return ::tpq::fail(code, __VA_ARGS__); \
    } while (0)

// Raises a kernel's dynamic LDS limit once per device; `done` is a bit per device id, one
// word per kernel instantiation.  Safe to call from several threads.
inline int ensure_dynamic_lds(const void* kernel, size_t bytes, std::atomic<uint64_t>& done, const char* what) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(TPQ_ERR_RUNTIME, "%s: no current device", what);
    const uint64_t bit = uint64_t{1} << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return TPQ_OK;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
    if (e != hipSuccess) return fail(TPQ_ERR_RUNTIME, "%s: cannot reserve %zu bytes of LDS: %s", what, bytes, hipGetErrorString(e));
    done.fetch_or(bit, std::memory_order_release);
    return TPQ_OK;
}

// Sweep knobs.  Environment variables named TPQ_* select kernels and workgroup shapes only in a build made with
// -DTPQ_TUNING (sweeps, comparison runs).  The shipped library never reads the environment: which kernel runs is a
// function of the arguments alone, and no entry point depends on getenv (not safe against a concurrent setenv).
inline const char* tuning_env(const char* name) {
#ifdef TPQ_TUNING
    return std::getenv(name);
#else
    (void)name;
    return nullptr;
#endif
}

// Routes that tests pin explicitly, so that a kernel is checked on every shape it can take and not only where the
// default rule sends it: -1 = the default rule.  They exist only in a build with -DTPQ_TEST_HOOKS (the library the
// tests' route-pinning fixture loads, with tpq_set_kernel_override exported); in the library that ships the kernel
// that runs depends on the arguments alone.
#ifdef TPQ_TEST_HOOKS
extern std::atomic<int> g_override_int8_row;    // 0 never / 1 up to four rows on the int8 row kernel
extern std::atomic<int> g_override_lowbit_row;  // 0 never / 1 wherever the shape allows, the packed n-bit row kernel
extern std::atomic<int> g_override_int4_row;    // 0 never / 1 wherever the shape allows, the int4 tile-streaming one-row kernel
inline int route_override_int8_row() { return g_override_int8_row.load(std::memory_order_relaxed); }
inline int route_override_lowbit_row() { return g_override_lowbit_row.load(std::memory_order_relaxed); }
inline int route_override_int4_row() { return g_override_int4_row.load(std::memory_order_relaxed); }
#else
inline int route_override_int8_row() { return -1; }
inline int route_override_lowbit_row() { return -1; }
inline int route_override_int4_row() { return -1; }
#endif

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// ---- 16-bit float conversions (bit patterns) ------------------------------

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(b) << 16);
}

// Round to nearest even; NaN becomes the quiet pattern 0x7FC0.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu) != 0) return 0x7FC0u;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    return static_cast<float>(__builtin_bit_cast(_Float16, h));
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));  // v_cvt_f16_f32: RNE
}

template <int DT>
struct Elem;
template <>
struct Elem<TPQ_DTYPE_F32> {
    using storage = float;
    static __device__ __forceinline__ float load(float v) { return v; }
    static __device__ __forceinline__ float store(float v) { return v; }
};
template <>
struct Elem<TPQ_DTYPE_F16> {
    using storage = uint16_t;
    static __device__ __forceinline__ float load(uint16_t v) { return f16_bits_to_f32(v); }
    static __device__ __forceinline__ uint16_t store(float v) { return f32_to_f16_bits(v); }
};
template <>
struct Elem<TPQ_DTYPE_BF16> {
    using storage = uint16_t;
    static __device__ __forceinline__ float load(uint16_t v) { return bf16_bits_to_f32(v); }
    static __device__ __forceinline__ uint16_t store(float v) { return f32_to_bf16_bits(v); }
};

// A global address whose origin the compiler has lost sight of: a load through it stays where it is written.  Loads
// through a __restrict__ const kernel argument may be moved down to their use, across barriers, which turns a fetch
// that was meant to travel under the main loop into a trip to memory in the epilogue.
template <class T>
__device__ __forceinline__ const __attribute__((address_space(1))) T* pinned_global(const T* p) {
    asm volatile("" : "+v"(p));
    return (const __attribute__((address_space(1))) T*)p;
}

// ---- streaming loads -------------------------------------------------------------------------

// Loads marked non-temporal, for data that is read once (weights): measured 7.2 -> 6.8 us on the
// int4 GEMV at 4096 x 11008.
__device__ __forceinline__ uint4 nt_load(const uint4* p) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const u4 v = __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 nt_load(const uint2* p) {
    typedef uint32_t u2 __attribute__((ext_vector_type(2)));
    const u2 v = __builtin_nontemporal_load(reinterpret_cast<const u2*>(p));
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t nt_load(const uint32_t* p) { return __builtin_nontemporal_load(p); }

// Every vector-memory load issued so far has landed (s_waitcnt vmcnt(0), as an instruction the compiler's own wait
// counting sees).  For the front of a loop whose body keeps loads in flight across the back edge: the wait counts the
// compiler puts inside a loop are the worst case over the ways into it, and with the prologue's loads still pending
// (asked for under conditions, in another order) every wait of the body becomes a wait for all outstanding loads,
// the ones just issued included.  With nothing pending on the way in the body's waits are exact.
// Worth 0.4 - 1.1 us in the packed n-bit matrix-core kernel; the int4 and int8 weight-only loop kernels, rebuilt the same
// way (branch-free steady loop, nothing pending on the way in), did not change.
__device__ __forceinline__ void drain_vector_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

__device__ __forceinline__ void nt_store(float4* p, float a, float b, float c, float d) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 v = {a, b, c, d};
    __builtin_nontemporal_store(v, reinterpret_cast<f4*>(p));
}

__device__ __forceinline__ void nt_store(uint4* p, const uint4& v) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const u4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<u4*>(p));
}

// ---- eight consecutive activations as floats ----------------------------------------------------

// p is 16-byte aligned (32 for fp32)
template <int DT>
__device__ __forceinline__ void load_eight(const typename Elem<DT>::storage* p, float (&v)[8]) {
    if constexpr (DT == TPQ_DTYPE_F32) {
        const float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        const uint4 raw = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = Elem<DT>::load(static_cast<uint16_t>(w[i] & 0xFFFFu));
            v[2 * i + 1] = Elem<DT>::load(static_cast<uint16_t>(w[i] >> 16));
        }
    }
}

// ---- 64-lane reductions -----------------------------------------------------

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

}  // namespace tpq
