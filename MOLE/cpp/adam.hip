// Fused Adam / AdamW update of one flat parameter array: one pass over p, g, m, v.
// Replaces the eleven tensor-op passes of _MOLECore::adam (MOLE/cpp/define.hpp:543-579), which
// instant_adam (MOLE/cpp/core.cpp:848-943) runs on the parameters, gradients and moments of a batch of
// offloaded experts between their fetch from pinned host memory and their write-back.
//
// HBM bound.  Bytes per element: fp32 parameters 16 read + 12 written; bf16 parameters (moments stay
// fp32) 12 read + 10 written.  Every thread moves 16-byte vectors; the arithmetic is fp32 without
// contraction into FMAs, in the reference's order of operations, so that it agrees with a
// tensor-op-by-tensor-op evaluation to the last bit or two.
#include "common.h"

namespace mole {

struct AdamArgs {
    float beta1, beta2, lr, lam, eps, bc1, bc2;   // bc = 1 - beta^t
    int adamw;
};

__device__ __forceinline__ void adam_one(float &p, float g, float &m, float &v, const AdamArgs &a) {
#pragma clang fp contract(off)
    if (a.adamw) p = p * (1.0f - a.lam * a.lr);
    else g = g + a.lam * p;
    m = a.beta1 * m + (1.0f - a.beta1) * g;
    v = a.beta2 * v + ((1.0f - a.beta2) * g) * g;
    const float mt = m / a.bc1, vt = v / a.bc2;
    p = p - (a.lr * mt) / (sqrtf(vt) + a.eps);
}

constexpr int ADAM_THREADS = 256;

// fp32 parameters: 4 elements per thread
__global__ __launch_bounds__(ADAM_THREADS) void adam_f32_kernel(const float *__restrict__ p, const float *__restrict__ g,
                                                                float *__restrict__ m, float *__restrict__ v,
                                                                float *__restrict__ p_out, size_t n, AdamArgs a) {
    const size_t i = ((size_t)blockIdx.x * ADAM_THREADS + threadIdx.x) * 4;
    if (i + 4 <= n) {
        float4 pp = *reinterpret_cast<const float4 *>(p + i);
        const float4 gg = *reinterpret_cast<const float4 *>(g + i);
        float4 mm = *reinterpret_cast<const float4 *>(m + i);
        float4 vv = *reinterpret_cast<const float4 *>(v + i);
        adam_one(pp.x, gg.x, mm.x, vv.x, a);
        adam_one(pp.y, gg.y, mm.y, vv.y, a);
        adam_one(pp.z, gg.z, mm.z, vv.z, a);
        adam_one(pp.w, gg.w, mm.w, vv.w, a);
        *reinterpret_cast<float4 *>(p_out + i) = pp;
        *reinterpret_cast<float4 *>(m + i) = mm;
        *reinterpret_cast<float4 *>(v + i) = vv;
    } else {
        for (size_t j = i; j < n; ++j) {
            float pp = p[j], mm = m[j], vv = v[j];
            adam_one(pp, g[j], mm, vv, a);
            p_out[j] = pp; m[j] = mm; v[j] = vv;
        }
    }
}

// bf16 parameters and gradients, fp32 moments: 8 elements per thread
__global__ __launch_bounds__(ADAM_THREADS) void adam_bf16_kernel(const bf16_t *__restrict__ p, const bf16_t *__restrict__ g,
                                                                 float *__restrict__ m, float *__restrict__ v,
                                                                 bf16_t *__restrict__ p_out, size_t n, AdamArgs a) {
    const size_t i = ((size_t)blockIdx.x * ADAM_THREADS + threadIdx.x) * 8;
    if (i + 8 <= n) {
        const uint4 pr = *reinterpret_cast<const uint4 *>(p + i);
        const uint4 gr = *reinterpret_cast<const uint4 *>(g + i);
        float mm[8], vv[8];
        *reinterpret_cast<float4 *>(mm) = *reinterpret_cast<const float4 *>(m + i);
        *reinterpret_cast<float4 *>(mm + 4) = *reinterpret_cast<const float4 *>(m + i + 4);
        *reinterpret_cast<float4 *>(vv) = *reinterpret_cast<const float4 *>(v + i);
        *reinterpret_cast<float4 *>(vv + 4) = *reinterpret_cast<const float4 *>(v + i + 4);
        const uint32_t pw[4] = {pr.x, pr.y, pr.z, pr.w}, gw[4] = {gr.x, gr.y, gr.z, gr.w};
        uint32_t ow[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float plo = __uint_as_float(pw[q] << 16), phi = __uint_as_float(pw[q] & 0xffff0000u);
            adam_one(plo, __uint_as_float(gw[q] << 16), mm[2 * q], vv[2 * q], a);
            adam_one(phi, __uint_as_float(gw[q] & 0xffff0000u), mm[2 * q + 1], vv[2 * q + 1], a);
            const bf16_t lo = (bf16_t)plo, hi = (bf16_t)phi;   // round to nearest even
            ow[q] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        *reinterpret_cast<uint4 *>(p_out + i) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
        *reinterpret_cast<float4 *>(m + i) = *reinterpret_cast<float4 *>(mm);
        *reinterpret_cast<float4 *>(m + i + 4) = *reinterpret_cast<float4 *>(mm + 4);
        *reinterpret_cast<float4 *>(v + i) = *reinterpret_cast<float4 *>(vv);
        *reinterpret_cast<float4 *>(v + i + 4) = *reinterpret_cast<float4 *>(vv + 4);
    } else {
        for (size_t j = i; j < n; ++j) {
            float pp = (float)p[j], mm = m[j], vv = v[j];
            adam_one(pp, (float)g[j], mm, vv, a);
            p_out[j] = (bf16_t)pp; m[j] = mm; v[j] = vv;
        }
    }
}

// acc[i] = acc[i] + add[i], rounded once to the parameter dtype (the reference's host-side `+=` of two tensors of that
// dtype, data_transfer.cpp:9-12): 16 bytes per lane in, 16 out.
template <typename T>
__global__ __launch_bounds__(ADAM_THREADS) void grad_add_kernel(T *__restrict__ acc, const T *__restrict__ add, size_t n) {
    constexpr int V = 16 / sizeof(T);
    const size_t i = ((size_t)blockIdx.x * ADAM_THREADS + threadIdx.x) * V;
    if (i + V <= n) {
        if constexpr (sizeof(T) == 4) {
            float4 a = *reinterpret_cast<const float4 *>(acc + i);
            const float4 b = *reinterpret_cast<const float4 *>(add + i);
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
            *reinterpret_cast<float4 *>(acc + i) = a;
        } else {
            const uint4 a = *reinterpret_cast<const uint4 *>(acc + i), b = *reinterpret_cast<const uint4 *>(add + i);
            const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
            uint32_t ow[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bf16_t lo = (bf16_t)(__uint_as_float(aw[q] << 16) + __uint_as_float(bw[q] << 16));
                const bf16_t hi = (bf16_t)(__uint_as_float(aw[q] & 0xffff0000u) + __uint_as_float(bw[q] & 0xffff0000u));
                ow[q] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
            }
            *reinterpret_cast<uint4 *>(acc + i) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
        }
    } else {
        for (size_t j = i; j < n; ++j) acc[j] = from_f32<T>(to_f32(acc[j]) + to_f32(add[j]));
    }
}

}  // namespace mole

using namespace mole;

extern "C" int mole_grad_add(void *acc, const void *add, size_t n, int dtype, mole_stream_t stream) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "mole_grad_add: bad dtype %d", dtype);
    if (n == 0) return 0;
    MOLE_REQUIRE(acc && add, "mole_grad_add: null pointer");
    MOLE_REQUIRE((((uintptr_t)acc | (uintptr_t)add) & 15) == 0, "mole_grad_add: buffers must be 16-byte aligned");
    const size_t per_block = (size_t)ADAM_THREADS * (dtype == MOLE_BF16 ? 8 : 4);
    const size_t blocks = (n + per_block - 1) / per_block;
    MOLE_REQUIRE(blocks <= 0x7fffffffull, "mole_grad_add: n=%zu too large for one launch", n);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MOLE_BF16)
        hipLaunchKernelGGL(grad_add_kernel<bf16_t>, dim3((unsigned)blocks), dim3(ADAM_THREADS), 0, st, (bf16_t *)acc, (const bf16_t *)add, n);
    else
        hipLaunchKernelGGL(grad_add_kernel<float>, dim3((unsigned)blocks), dim3(ADAM_THREADS), 0, st, (float *)acc, (const float *)add, n);
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" int mole_adam_step(const void *p, const void *g, float *m, float *v, void *p_out, size_t n, int dtype,
                              float beta1, float beta2, int t, float lr, float lam, float eps, int adamw,
                              mole_stream_t stream) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "mole_adam_step: bad dtype %d", dtype);
    MOLE_REQUIRE(t >= 1, "mole_adam_step: step count t=%d must be >= 1 (the reference passes its counter + 1)", t);
    if (n == 0) return 0;
    MOLE_REQUIRE(p && g && m && v && p_out, "mole_adam_step: null pointer");
    MOLE_REQUIRE((((uintptr_t)p | (uintptr_t)g | (uintptr_t)m | (uintptr_t)v | (uintptr_t)p_out) & 15) == 0,
                 "mole_adam_step: buffers must be 16-byte aligned");
    AdamArgs a;
    a.beta1 = beta1; a.beta2 = beta2; a.lr = lr; a.lam = lam; a.eps = eps; a.adamw = adamw;
    // 1 - std::pow(beta, t) is a double in the reference and becomes a float scalar of the tensor division
    a.bc1 = (float)(1.0 - pow((double)beta1, (double)t));
    a.bc2 = (float)(1.0 - pow((double)beta2, (double)t));
    MOLE_REQUIRE(a.bc1 > 0.f && a.bc2 > 0.f, "mole_adam_step: beta1=%g beta2=%g must be below 1", beta1, beta2);
    const int per_thread = dtype == MOLE_BF16 ? 8 : 4;
    const size_t per_block = (size_t)ADAM_THREADS * per_thread;
    const size_t blocks = (n + per_block - 1) / per_block;
    MOLE_REQUIRE(blocks <= 0x7fffffffull, "mole_adam_step: n=%zu too large for one launch", n);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MOLE_BF16)
        timed_launch(MOLE_K_ADAM, adam_bf16_kernel, dim3((unsigned)blocks), dim3(ADAM_THREADS), 0, st, (const bf16_t *)p,
                     (const bf16_t *)g, m, v, (bf16_t *)p_out, n, a);
    else
        timed_launch(MOLE_K_ADAM, adam_f32_kernel, dim3((unsigned)blocks), dim3(ADAM_THREADS), 0, st, (const float *)p,
                     (const float *)g, m, v, (float *)p_out, n, a);
    MOLE_LAUNCH_CHECK();
    return 0;
}
