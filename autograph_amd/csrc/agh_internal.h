// Shared internals of the C-ABI library: error reporting, the single stream, the
// library-owned workspace, argument checks and device-side bf16 helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "../../include/autograph_hip.h"

namespace agh {

// One lock serialises every entry point (the reference's tensors are Send + Sync and
// krnl queues work in order per device).
std::recursive_mutex &api_mutex();
hipStream_t stream();
bool initialized();
int compute_units();
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char *what);
// Scratch owned by the library (split-K partials); grows on demand, never shrinks.
int workspace(size_t bytes, void **ptr);
// The fixed scratch buffer of agh_gemm_bf16_noalloc instead: never allocates, fails beyond its size.
int static_workspace(size_t bytes, void **ptr);
// Conv2 forward as an implicit GEMM (agh_conv_mfma.hip), T = uint16_t (bf16) or float; 1 = geometry not taken,
// else a status code
template <typename T>
int conv2_mfma_try(const char *name, const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic, int64_t ih,
                   int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t oh, int64_t ow, int act);

#define AGH_API_ENTER()                                           \
    std::lock_guard<std::recursive_mutex> _agh_lock(agh::api_mutex()); \
    if (!agh::initialized()) return agh::fail(AGH_ENOINIT, "%s: agh_init has not been called", __func__)

#define AGH_HIP(expr)                                                  \
    do {                                                               \
        hipError_t _e = (expr);                                        \
        if (_e != hipSuccess) return agh::hip_fail(_e, #expr);         \
    } while (0)

#define AGH_LAUNCH_CHECK(name)                                         \
    do {                                                               \
        hipError_t _e = hipGetLastError();                             \
        if (_e != hipSuccess) return agh::hip_fail(_e, name);          \
    } while (0)

// Division by a launch-constant divisor d (1 <= d < 2^31) of values n < 2^31 with one
// multiply-high, an add and a shift.
struct FastDiv {
    uint32_t d, magic, shift;
    FastDiv() : d(1), magic(0), shift(0) {}
    explicit FastDiv(uint32_t div) : d(div) {
        for (shift = 0; shift < 32; ++shift)
            if ((1u << shift) >= d) break;
        uint64_t one = 1;
        magic = (uint32_t)(((one << 32) * ((one << shift) - d)) / d + 1);
    }
    __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        return (__umulhi(n, magic) + n) >> shift;
#else
        return (uint32_t)((((uint64_t)n * magic) >> 32) + n) >> shift;
#endif
    }
    __host__ __device__ __forceinline__ void divmod(uint32_t n, uint32_t &q, uint32_t &r) const {
        q = div(n);
        r = n - q * d;
    }
};

// ---- bf16 <-> f32 exactly as the `half` crate does it (the reference's bf16 type) ----
// (written with selects, not branches: these sit in GEMM epilogues and per-element loops)
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
    const uint32_t x = (uint32_t)h << 16;
    const bool nan = (h & 0x7FFFu) > 0x7F80u;
    return __uint_as_float(nan ? (x | 0x00400000u) : x);  // NaN: set the quiet bit
}
// f32 -> bf16, round to nearest even, NaN -> (x >> 16) | 0x40.  gfx950 has this as an instruction
// (v_cvt_pk_bf16_f32, which the conversion below compiles to); it agrees with the `half` crate's
// rule on every f32 whose low half is one of 0, 1, 0x4000, 0x7FFF, 0x8000, 0x8001, 0xC000, 0xFFFF
// for all 65536 high halves (ties, NaNs with any payload, infinities, subnormals): checked on the device.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
// two at once: low half = a, high half = b
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t in = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(in, bf16x2_t));
}
// widening without the NaN quieting of bf16_to_f32: for values that go straight into an addition
// (which quiets a signalling NaN itself) or that this library has just rounded (already quiet)
__device__ __forceinline__ float bf16_raw_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float to_f32(float v) { return v; }
    static __device__ __forceinline__ float raw(float v) { return v; }
    static __device__ __forceinline__ float from_f32(float v) { return v; }
    static __device__ __forceinline__ float zero() { return 0.0f; }
};
template <> struct Elem<uint16_t> {
    static __device__ __forceinline__ float to_f32(uint16_t v) { return bf16_to_f32(v); }
    // the plain widening, for an operand of an addition or a comparison: the addition quiets a signalling NaN
    // itself, and a comparison with any NaN is false either way
    static __device__ __forceinline__ float raw(uint16_t v) { return bf16_raw_f32(v); }
    static __device__ __forceinline__ uint16_t from_f32(float v) { return f32_to_bf16(v); }
    static __device__ __forceinline__ uint16_t zero() { return 0; }
};

}  // namespace agh
