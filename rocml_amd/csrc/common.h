// Shared helpers of the HIP sources: error reporting, dtype codes, bf16 conversion,
// wave64 reductions.  Every exported function returns 0 on success; on failure it
// returns nonzero and leaves a message that <family>_last_error() returns, the way
// the reference's HIP layer turns a status into code + message
// (rocml-hip/src/error.rs:32-48).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#define ROCML_EXPORT extern "C" __attribute__((visibility("default")))

enum RocmlDtype : int { ROCML_F32 = 0, ROCML_BF16 = 1 };

static thread_local char g_rocml_err[1024] = "";

static int rocml_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_rocml_err, sizeof(g_rocml_err), fmt, ap);
    va_end(ap);
    return 1;
}

#define ROCML_REQUIRE(cond, ...)                       \
    do {                                               \
        if (!(cond)) return rocml_fail(__VA_ARGS__);   \
    } while (0)

#define ROCML_CHECK_LAUNCH(name)                                                         \
    do {                                                                                 \
        hipError_t e_ = hipGetLastError();                                               \
        if (e_ != hipSuccess)                                                            \
            return rocml_fail("%s: launch failed: %s (%d)", name, hipGetErrorString(e_), \
                              (int)e_);                                                  \
    } while (0)

#define ROCML_LAST_ERROR_FN(family) \
    ROCML_EXPORT const char* family##_last_error() { return g_rocml_err; }

// Compute units of the current device (256 on an MI355X).  Launch sizes are phrased in it: how
// many blocks fill the chip, how many tiles leave CUs idle.
static int cu_count() {
    static int cached[64] = {0};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
    if (cached[device] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) n = 256;
        cached[device] = n;
    }
    return cached[device];
}

// ---- bf16 as raw 16 bits ------------------------------------------------------
typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// Round to nearest even; NaN stays NaN.  gfx950 has the conversion in hardware
// (v_cvt_pk_bf16_f32), which the compiler picks for these casts.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }

// two values in one instruction: a in the low half
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_t_;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t_;
    f32x2_t_ v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t_));
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
    static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
    static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
};

// ---- wave64 reductions --------------------------------------------------------
constexpr int WAVE = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

static inline int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }
