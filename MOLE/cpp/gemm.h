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
__device__ __forceinline__ float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f)); }

// derivative of the tanh-approximate GELU, term by term as MOLE/cpp/gelu.cu:3-14
__device__ __forceinline__ float d_gelu_tanh(float x) {
    const float sqrt_param = 0.79788456080286535587989211986876f;
    const float mul_param = 0.044715f;
    const float x2mul = x * x * mul_param;
    const float tan_h = tanhf(sqrt_param * (x + x * x2mul));
    const float dg1 = 0.5f * (1.0f + tan_h);
    const float dg2 = x * 0.5f * sqrt_param * (1.0f - tan_h * tan_h);
    const float dg3 = dg2 * 3.0f * x2mul;
    return dg1 + dg2 + dg3;
}
// derivative of the erf GELU (at::gelu_backward): Phi(x) + x*phi(x)
__device__ __forceinline__ float d_gelu_exact(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752f));
    const float pdf = expf(-0.5f * x * x) * 0.39894228040143267794f;
    return cdf + x * pdf;
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
    void *colsum;           // weight gradients, 256-wide kernel: [E][M] (side 1) or [E][N] (side 2) sums of an operand
    int colsum_side;        //   over the expert's rows: 1 = the m-side operand (A), 2 = the n-side operand (B)
    int wg_expert_major;    // weight gradients, 256-wide kernel: all (m-tile, n-tile) blocks of an expert on one XCD
    int m_fastest;          // row-ragged products, 256-wide kernel: number an expert's tiles m-tile first (see gemm256.hip)
};


// 256x256 bf16 tiles with direct-to-LDS loads (gemm256.hip).  Returns -100 when the shape does not
// meet its alignment requirements; the caller then uses the generic kernel.
int launch_gemm256(const GemmArgs &g, bool a_ks, bool b_ks, bool wg, int epi, int max_rows, hipStream_t st, int kid);
bool gemm256_sums_operand(const GemmArgs &g, int kid);

}  // namespace mole
