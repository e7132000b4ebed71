// Internal helpers shared by the translation units of libpipedream_amd.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "pipedream_amd.h"

// Thread-local last-error message (pd_last_error()).
void pd_set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define PD_FAIL(code, ...)        \
    do {                          \
        pd_set_error(__VA_ARGS__);\
        return (code);            \
    } while (0)

#define PD_REQUIRE(cond, code, ...) \
    do {                            \
        if (!(cond)) PD_FAIL(code, __VA_ARGS__); \
    } while (0)

// Check the launch that was just issued; returns the hipError_t on failure.
#define PD_CHECK_LAUNCH(name)                                             \
    do {                                                                  \
        hipError_t e__ = hipGetLastError();                               \
        if (e__ != hipSuccess) {                                          \
            pd_set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
            return (int)e__;                                              \
        }                                                                 \
    } while (0)

#define PD_HIP(call)                                                      \
    do {                                                                  \
        hipError_t e__ = (call);                                          \
        if (e__ != hipSuccess) {                                          \
            pd_set_error("%s failed: %s", #call, hipGetErrorString(e__)); \
            return (int)e__;                                              \
        }                                                                 \
    } while (0)

static inline bool pd_aligned(const void* p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// 64-lane wavefronts on gfx950.
#define PD_WAVE 64

#if defined(__HIPCC__)
// fp32 -> bf16, round to nearest even: the gfx950 conversion instruction (v_cvt_pk_bf16_f32; the
// compiler pairs two adjacent conversions into one instruction).
__device__ __forceinline__ uint16_t pd_f2bf(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
#endif
