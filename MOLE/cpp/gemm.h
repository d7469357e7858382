// Shared declarations of the grouped-GEMM kernels: argument block, epilogue kinds, activation math.
#pragma once
#include "common.h"

#include <math.h>

namespace mole {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// ---------------------------------------------------------------------------------------------
// activation math (fp32)
// ---------------------------------------------------------------------------------------------
// Phi(x) = 1/2 (1 + erf(x / sqrt 2)) and exp(-x^2 / 2), from one hardware exponential and one reciprocal: erf by the
// rational form of Abramowitz & Stegun 7.1.26 (absolute error 1.5e-7), written for the tail that is small so that
// nothing cancels: Phi(x) = q for x < 0 and 1 - q for x >= 0 with q = 1/2 t (a1 + t (a2 + ...)) exp(-x^2 / 2),
// t = 1 / (1 + p |x| / sqrt 2).  The library's erff costs about twice the instructions of everything else in an
// fp32 epilogue.
__device__ __forceinline__ float std_normal_cdf(float x, float &exp_half_sq) {
    const float y = fabsf(x) * 0.70710678118654752f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, y, 1.0f));
    float p = 1.061405429f;
    p = fmaf(p, t, -1.453152027f);
    p = fmaf(p, t, 1.421413741f);
    p = fmaf(p, t, -0.284496736f);
    p = fmaf(p, t, 0.254829592f);
    exp_half_sq = __builtin_amdgcn_exp2f(-y * y * 1.44269504088896341f);
    const float q = 0.5f * p * t * exp_half_sq;
    return x < 0.f ? q : 1.0f - q;
}
__device__ __forceinline__ float gelu_erf(float x) {
    float e;
    return x * std_normal_cdf(x, e);
}

// derivative of the tanh-approximate GELU, term by term as MOLE/cpp/gelu.cu:3-14; tanh(u) = 1 - 2 / (1 + exp(2u)),
// which saturates correctly at both ends (exp -> inf gives 1, exp -> 0 gives -1)
__device__ __forceinline__ float d_gelu_tanh(float x) {
    const float sqrt_param = 0.79788456080286535587989211986876f;
    const float mul_param = 0.044715f;
    const float x2mul = x * x * mul_param;
    const float u = sqrt_param * (x + x * x2mul);
    // exp(2u) = 2^(hi) (1 + lo ln 2): hi + lo is the product 2u log2(e) to twice the working precision (at |u| of a few
    // units the rounding of the product alone would cost a digit of the exponential)
    const float c_hi = 2.88539008177792681f, c_lo = 2.88539008177792681 - (double)c_hi;
    const float hi = u * c_hi;
    const float lo = fmaf(u, c_hi, -hi) + u * c_lo;
    const float e2u = __builtin_amdgcn_exp2f(hi) * fmaf(lo, 0.69314718055994531f, 1.0f);
    const float tan_h = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e2u);
    const float dg1 = 0.5f * (1.0f + tan_h);
    const float dg2 = x * 0.5f * sqrt_param * (1.0f - tan_h * tan_h);
    const float dg3 = dg2 * 3.0f * x2mul;
    return dg1 + dg2 + dg3;
}
// derivative of the erf GELU (at::gelu_backward): Phi(x) + x*phi(x)
__device__ __forceinline__ float d_gelu_exact(float x) {
    float e;
    const float cdf = std_normal_cdf(x, e);
    return cdf + x * e * 0.39894228040143267794f;
}

enum { EPI_STORE = 0, EPI_BIAS = 1, EPI_BIAS_GELU = 2, EPI_DGELU = 3, EPI_WGRAD = 4, EPI_F32 = 5,
       EPI_NONE = 6 /* measurement only: the K loop runs, nothing is stored; EPI_NONE + 1..4: the K loop without
                       its operand loads / its fragment reads / its barriers / all three */ };

struct GemmArgs {
    const void *A, *B;      // operands (see A_KS / B_KS for their layout)
    void *C, *C2;           // outputs; C2 = gelu(h) for EPI_BIAS_GELU
    const void *bias;       // [E][N] for EPI_BIAS*, else unused
    const void *H;          // [rows][N] pre-activation for EPI_DGELU
    const int32_t *offsets; // [E] first row of every expert (NULL: one group starting at row 0)
    const int32_t *kept;    // [E] rows of every expert (NULL: single_rows)
    int single_rows;
    int E;
    int M;                  // output rows per expert for weight gradients (F), unused for row-ragged
    int N, K;               // N output columns; K contraction length (row-ragged products)
    long lda, ldb, ldc;
    long strideB;           // elements between experts in B (row-ragged) -- weights
    long strideC;           // elements between experts in C (weight gradients)
    int m_tiles_bound;      // upper bound of the number of m-tiles over all experts (row-ragged)
    int accumulate;         // EPI_WGRAD: add into C
    int gelu_bwd;           // EPI_DGELU: MOLE_GELU_BWD_*
    int n_blocks;           // real number of tiles in the launch (grid is rounded up to 8)
    void *colsum;           // weight gradients, direct-to-LDS kernels: [E][M] (side 1) or [E][N] (side 2) sums of an operand
    int colsum_side;        //   over the expert's rows: 1 = the m-side operand (A), 2 = the n-side operand (B)
    int wg_expert_major;    // weight gradients, 256-wide kernel: all (m-tile, n-tile) blocks of an expert on one XCD
    int m_fastest_from;     //   ... for experts with at least this many m-tiles (of the class); the others n-tile first
    int m_fastest;          // row-ragged products, 256-wide kernel: number an expert's tiles m-tile first (see gemm256.hip)
};


// 256x256 bf16 tiles with direct-to-LDS loads (gemm256.hip).  Returns -100 when the shape does not
// meet its alignment requirements; the caller then uses the generic kernel.
int launch_gemm256(const GemmArgs &g, bool a_ks, bool b_ks, bool wg, int epi, int max_rows, hipStream_t st, int kid);
bool gemm256_sums_operand(const GemmArgs &g, int kid);
// fp32 tiles with direct-to-LDS loads (gemm_f32.hip); -100 as above.
int launch_gemm_f32(const GemmArgs &g, bool a_ks, bool b_ks, bool wg, int epi, int max_rows, hipStream_t st, int kid);
bool gemm_f32_sums_operand(const GemmArgs &g);

}  // namespace mole
