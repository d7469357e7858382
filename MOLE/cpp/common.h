// Shared helpers of the gfx950 kernels: error plumbing, bf16 <-> fp32, wave-level primitives.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "mole_hip.h"

namespace mole {

void set_error(const char *fmt, ...);

#define MOLE_REQUIRE(cond, ...)                 \
    do {                                        \
        if (!(cond)) {                          \
            mole::set_error(__VA_ARGS__);       \
            return MOLE_E_INVALID;              \
        }                                       \
    } while (0)

#define MOLE_HIP(call)                                                                   \
    do {                                                                                 \
        hipError_t e_ = (call);                                                          \
        if (e_ != hipSuccess) {                                                          \
            mole::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
            return (int)e_;                                                              \
        }                                                                                \
    } while (0)

// after a kernel launch: report launch-configuration errors without synchronising
#define MOLE_LAUNCH_CHECK()                                                              \
    do {                                                                                 \
        hipError_t e_ = hipGetLastError();                                               \
        if (e_ != hipSuccess) {                                                          \
            mole::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(e_), __FILE__, __LINE__); \
            return (int)e_;                                                              \
        }                                                                                \
    } while (0)

typedef __bf16 bf16_t;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }  // round to nearest even

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t lo16) { return __uint_as_float(lo16 << 16); }

constexpr int WAVE = 64;

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = WAVE / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, WAVE);
    return v;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// optional per-kernel timing (see error.cpp); ids are the MOLE_K_* of mole_hip.h
bool timing_enabled();
void timing_begin(int id, hipStream_t st);
void timing_end(hipStream_t st);
struct ScopedTiming {
    hipStream_t st;
    bool on;
    ScopedTiming(int id, hipStream_t s) : st(s), on(timing_enabled()) { if (on) timing_begin(id, st); }
    ~ScopedTiming() { if (on) timing_end(st); }
};

// One kernel under a timing id.  With timing on, the launch carries its own start/stop events, which take the
// kernel's begin and end from its dispatch packet: the measured time is the kernel's run time, as a profiler
// sees it.  (An event pair recorded around a launch adds two marker packets to the stream, about 2.4 us - a
// fifth of a 12 us kernel.)  ScopedTiming remains for entry points that launch several kernels under one id.
void timing_events(int id, hipEvent_t *start, hipEvent_t *stop);
template <typename... KArgs, typename... Args>
inline void timed_launch(int id, void (*kernel)(KArgs...), dim3 grid, dim3 block, unsigned lds, hipStream_t st,
                         Args... args) {
    if (timing_enabled()) {
        hipEvent_t a, b;
        timing_events(id, &a, &b);
        hipExtLaunchKernelGGL(kernel, grid, block, lds, st, a, b, 0, static_cast<KArgs>(args)...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds, st, static_cast<KArgs>(args)...);
    }
}

}  // namespace mole
