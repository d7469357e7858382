// Measurement aids for the grouped GEMM's roofline: what the matrix cores of this chip sustain on their own, and what
// the product's K loop sustains without an epilogue.  Not part of the MoE path (no counterpart in the reference); the
// benchmark script runs them so that the ceilings quoted beside the products' figures come from tracked code.
//
//   mole_probe_mfma   every wave issues v_mfma_f32_32x32x16_bf16 back to back on operands it holds in registers
//                     (eight waves per block, one block per CU, 128 accumulator registers per lane: the product's
//                     own register blocking), no memory traffic inside the loop.  Operands come from a caller
//                     buffer: zeros show the published peak, random data what the chip sustains under load.
//   mole_probe_kloop  the product kernel itself at a row-ragged shape (C = A . B^T, both K-contiguous, like
//                     h = xd . w1^T) with the epilogue left out: prologue + K loop (LDS-DMA feed, fragment reads,
//                     MFMAs) + launch.
#include "gemm.h"
#include "mole_hip_probe.h"

namespace mole {

constexpr int PROBE_THREADS = 512;

__global__ __launch_bounds__(PROBE_THREADS, 1) void probe_mfma_kernel(const uint4 *__restrict__ operands, int iters,
                                                                      float *__restrict__ sink) {
    extern __shared__ char smem[];     // sized by the launch so that one block fills a CU, as the product's does
    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
    bf16x8 m[4], n[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) m[i] = __builtin_bit_cast(bf16x8, operands[i * PROBE_THREADS + threadIdx.x]);
#pragma unroll
    for (int j = 0; j < 2; ++j) n[j] = __builtin_bit_cast(bf16x8, operands[(4 + j) * PROBE_THREADS + threadIdx.x]);
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(n[j], m[i], acc[i][j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) s += acc[i][j][0];
    if (iters < 0) smem[threadIdx.x] = 1;
    sink[(size_t)blockIdx.x * PROBE_THREADS + threadIdx.x] = s;
}

}  // namespace mole

using namespace mole;

extern "C" size_t mole_probe_mfma_operand_bytes(void) { return (size_t)6 * PROBE_THREADS * sizeof(uint4); }

extern "C" int mole_probe_mfma(const void *operands, int blocks, int iters, float *sink, double *flop_out,
                               mole_stream_t stream) {
    MOLE_REQUIRE(operands && sink && blocks > 0 && iters > 0, "mole_probe_mfma: bad arguments (blocks=%d iters=%d)", blocks, iters);
    const int lds = 128 * 1024;
    static bool attr_done = false;
    if (!attr_done) {
        MOLE_HIP(hipFuncSetAttribute((const void *)probe_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        attr_done = true;
    }
    timed_launch(MOLE_K_PROBE, probe_mfma_kernel, dim3(blocks), dim3(PROBE_THREADS), lds, (hipStream_t)stream,
                 (const uint4 *)operands, iters, sink);
    MOLE_LAUNCH_CHECK();
    // 8 MFMAs of 32 x 32 x 16 (2 x 16384 flop) per wave and iteration, 8 waves per block
    if (flop_out) *flop_out = (double)blocks * 8.0 * iters * 8.0 * 32768.0;
    return 0;
}

extern "C" int mole_probe_kloop_part(const void *a, const void *b, const int32_t *offsets, const int32_t *kept_rows, int E,
                                     int max_rows, int N, int K, int part, float *sink, mole_stream_t stream) {
    MOLE_REQUIRE(part >= 0 && part <= 4, "mole_probe_kloop_part: part %d is not one of 0..4", part);
    MOLE_REQUIRE(a && b && offsets && kept_rows && sink && E >= 1 && max_rows > 0 && N > 0 && K > 0 && N % 8 == 0 && K % 32 == 0,
                 "mole_probe_kloop: bad arguments (E=%d rows=%d N=%d K=%d)", E, max_rows, N, K);
    GemmArgs g{};
    g.offsets = offsets; g.kept = kept_rows; g.E = E;
    g.A = a; g.lda = K; g.B = b; g.ldb = K; g.strideB = (long)N * K; g.N = N; g.K = K; g.C = sink; g.ldc = N;
    const int rc = launch_gemm256(g, false, false, false, EPI_NONE + part, max_rows, (hipStream_t)stream, MOLE_K_PROBE);
    MOLE_REQUIRE(rc != -100, "mole_probe_kloop: shape not taken by the 256-wide kernel");
    return rc;
}

extern "C" int mole_probe_kloop(const void *a, const void *b, const int32_t *offsets, const int32_t *kept_rows, int E,
                                int max_rows, int N, int K, float *sink, mole_stream_t stream) {
    return mole_probe_kloop_part(a, b, offsets, kept_rows, E, max_rows, N, K, 0, sink, stream);
}
