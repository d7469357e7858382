// Dispatch scatter, combine gather and their backward: HBM-bound row permutes.
//
// Replaces tutel's fast_encode / fast_decode (GatingEncoder / GatingDecoder forward and backward;
// call sites MOLE/moe/layer.py:448-449 and 457-458).  One wave owns one token: it reads the
// token's k destination rows once (wave-uniform), then streams the row in 16-byte pieces per lane,
// so every global access is a full 1 KiB wave transaction.  The source row is read once and
// written k times (dispatch), or k rows are read and one written (combine); all sums are fp32.
#include "common.h"

#include <type_traits>

namespace mole {

template <typename T> struct Vec;  // 16 bytes of T
template <> struct Vec<float> {
    static constexpr int N = 4;
    float4 raw;
    __device__ __forceinline__ void load(const float *p) { raw = *reinterpret_cast<const float4 *>(p); }
    __device__ __forceinline__ void load_nt(const float *p) {       // read once: do not keep it in the caches
        typedef float f32x4_ __attribute__((ext_vector_type(4)));
        const f32x4_ w = __builtin_nontemporal_load(reinterpret_cast<const f32x4_ *>(p));
        raw = make_float4(w[0], w[1], w[2], w[3]);
    }
    __device__ __forceinline__ void store(float *p) const { *reinterpret_cast<float4 *>(p) = raw; }
    __device__ __forceinline__ void unpack(float *f) const { f[0] = raw.x; f[1] = raw.y; f[2] = raw.z; f[3] = raw.w; }
    __device__ __forceinline__ void pack(const float *f) { raw = make_float4(f[0], f[1], f[2], f[3]); }
    __device__ __forceinline__ void zero() { raw = make_float4(0.f, 0.f, 0.f, 0.f); }
    // makes the loaded value opaque to the compiler at this point: without it a load whose only uses sit under
    // branches is repeated inside every one of them, each time followed by a full wait
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(raw.x), "+v"(raw.y), "+v"(raw.z), "+v"(raw.w)); }
    __device__ __forceinline__ void mask(uint32_t m) {        // m = all ones (keep) or 0 (becomes +0)
        raw = make_float4(__uint_as_float(__float_as_uint(raw.x) & m), __uint_as_float(__float_as_uint(raw.y) & m),
                          __uint_as_float(__float_as_uint(raw.z) & m), __uint_as_float(__float_as_uint(raw.w) & m));
    }
};
template <> struct Vec<bf16_t> {
    static constexpr int N = 8;
    uint4 raw;
    __device__ __forceinline__ void load(const bf16_t *p) { raw = *reinterpret_cast<const uint4 *>(p); }
    __device__ __forceinline__ void load_nt(const bf16_t *p) {      // read once: do not keep it in the caches
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
        raw = make_uint4(w[0], w[1], w[2], w[3]);
    }
    __device__ __forceinline__ void store(bf16_t *p) const { *reinterpret_cast<uint4 *>(p) = raw; }
    __device__ __forceinline__ void unpack(float *f) const {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ __forceinline__ void pack(const float *f) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bf16_t lo = (bf16_t)f[2 * i], hi = (bf16_t)f[2 * i + 1];
            w[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        raw = make_uint4(w[0], w[1], w[2], w[3]);
    }
    __device__ __forceinline__ void zero() { raw = make_uint4(0, 0, 0, 0); }
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(raw.x), "+v"(raw.y), "+v"(raw.z), "+v"(raw.w)); }
    __device__ __forceinline__ void mask(uint32_t m) { raw = make_uint4(raw.x & m, raw.y & m, raw.z & m, raw.w & m); }
};

constexpr int PM_THREADS = 256;  // 4 waves = 4 tokens per block

// How these kernels keep memory busy.  A wave's loads are issued unconditionally, from addresses clamped to
// something valid, and a value that must not count (a dropped pair, a choice past k, a chunk past the row's end)
// is cleared with a bit mask where it is used.  A load written under a condition ("r >= 0 ? load : 0") compiles
// to a branch around the load, and the compiler then waits for every outstanding load at each such branch: the k
// row fetches of a token ran one after the other.  With K (the template's bound on k) x PM_U chunk loads in
// flight per wave the gathers reach the rate of a plain copy.
constexpr int PM_U = 2;          // 1 KiB chunks of a row in flight per wave and source row

// destination/source rows of token i for the K choice slots: row index (0 when the slot does not count) and
// keep mask (all ones when it does: a choice below k whose pair was kept)
template <int K>
__device__ __forceinline__ void load_rows(const int32_t *__restrict__ row, int S, int k, int i, int (&r)[K],
                                          uint32_t (&keep)[K]) {
#pragma unroll
    for (int j = 0; j < K; ++j) r[j] = row[(size_t)min(j, k - 1) * S + i];      // all K loads first
#pragma unroll
    for (int j = 0; j < K; ++j) {
        keep[j] = (j < k && r[j] >= 0) ? 0xffffffffu : 0u;
        r[j] &= (int)keep[j];
    }
}

// TPW tokens per wave: the row indices of all of a wave's tokens come first, then the loads of all their rows' pieces,
// then the stores.  A wave that owns a single token with a single choice has little in flight and pays the index
// latency once per row.
template <int K, int TPW>
__device__ __forceinline__ void load_rows_multi(const int32_t *__restrict__ row, int S, int k, int i0, int (&r)[TPW][K],
                                                uint32_t (&keep)[TPW][K]) {
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int j = 0; j < K; ++j) r[t][j] = row[(size_t)min(j, k - 1) * S + min(i0 + t, S - 1)];      // all loads first
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int j = 0; j < K; ++j) {
            keep[t][j] = (j < k && i0 + t < S && r[t][j] >= 0) ? 0xffffffffu : 0u;
            r[t][j] &= (int)keep[t][j];
        }
}

template <typename T, int K, int TPW>
__global__ __launch_bounds__(PM_THREADS) void dispatch_fwd_kernel(const T *__restrict__ x,
                                                                  const int32_t *__restrict__ row, int S, int M,
                                                                  int k, T *__restrict__ xd) {
    const int i0 = (blockIdx.x * (PM_THREADS / WAVE) + (threadIdx.x >> 6)) * TPW;
    if (i0 >= S) return;
    const int lane = lane_id();
    int r[TPW][K];
    uint32_t keep[TPW][K];
    load_rows_multi<K, TPW>(row, S, k, i0, r, keep);
    constexpr int N = Vec<T>::N;
    constexpr int U = TPW > 1 ? PM_U : 2 * PM_U;                  // one source row: more of its chunks in flight
    const int chunks = M / N;
    for (int c0 = lane; c0 < chunks; c0 += U * WAVE) {
        Vec<T> v[TPW][U];
#pragma unroll
        for (int t = 0; t < TPW; ++t)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * WAVE;
                v[t][u].load(x + (size_t)min(i0 + t, S - 1) * M + (size_t)(c < chunks ? c : c0) * N);
            }
#pragma unroll
        for (int t = 0; t < TPW; ++t)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * WAVE;
                v[t][u].pin();
                if (c < chunks) {
#pragma unroll
                    for (int j = 0; j < K; ++j)
                        if (keep[t][j]) v[t][u].store(xd + (size_t)r[t][j] * M + (size_t)c * N);
                }
            }
    }
}

template <typename T, int K>
__global__ __launch_bounds__(PM_THREADS) void dispatch_bwd_kernel(const T *__restrict__ dxd,
                                                                  const int32_t *__restrict__ row, int S, int M,
                                                                  int k, const float *__restrict__ dlogits,
                                                                  const float *__restrict__ wg, int E,
                                                                  const T *__restrict__ dx_add, T *__restrict__ dx) {
    const int i = blockIdx.x * (PM_THREADS / WAVE) + (threadIdx.x >> 6);
    if (i >= S) return;
    const int lane = lane_id();
    int r[K];
    uint32_t keep[K];
    load_rows<K>(row, S, k, i, r, keep);
    constexpr int N = Vec<T>::N;
    constexpr int U = K >= 16 ? 1 : PM_U;
    const int chunks = M / N;
    // the optional addend goes through the same path as one more source row (row i of dx_add, or masked out)
    const T *add_row = dx_add != nullptr ? dx_add + (size_t)i * M : dxd;
    const uint32_t add_keep = dx_add != nullptr ? 0xffffffffu : 0u;
    for (int c0 = lane; c0 < chunks; c0 += U * WAVE) {
        Vec<T> v[U][K], va[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + u * WAVE;
            const size_t off = (size_t)(c < chunks ? c : c0) * N;
#pragma unroll
            for (int j = 0; j < K; ++j) v[u][j].load(dxd + (size_t)r[j] * M + off);
            va[u].load(add_row + off);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + u * WAVE;
            if (c >= chunks) continue;
            float acc[N], f[N];
#pragma unroll
            for (int q = 0; q < N; ++q) acc[q] = 0.f;
#pragma unroll
            for (int j = 0; j < K; ++j) {
                v[u][j].mask(keep[j]);
                v[u][j].unpack(f);
#pragma unroll
                for (int q = 0; q < N; ++q) acc[q] += f[q];
            }
            va[u].mask(add_keep);
            va[u].unpack(f);
#pragma unroll
            for (int q = 0; q < N; ++q) acc[q] += f[q];
            if (dlogits != nullptr) {
                for (int e = 0; e < E; ++e) {
                    const float dl = dlogits[(size_t)i * E + e];
                    const float *wrow = wg + (size_t)e * M + (size_t)c * N;
#pragma unroll
                    for (int q = 0; q < N; q += 4) {
                        const float4 wv = *reinterpret_cast<const float4 *>(wrow + q);
                        acc[q] += dl * wv.x;
                        acc[q + 1] += dl * wv.y;
                        acc[q + 2] += dl * wv.z;
                        acc[q + 3] += dl * wv.w;
                    }
                }
            }
            Vec<T> o;
            o.pack(acc);
            o.store(dx + (size_t)i * M + (size_t)c * N);
        }
    }
}

// dispatch backward with the gate's input gradient folded in, for small gates (E <= 32): a thread
// owns 4 columns and keeps its 4 x E slice of Wg in registers; the block walks db_tokens tokens (8 or 32), whose
// row indices and dlogits are block-uniform (scalar loads).  Larger gates use the kernel above.
constexpr int DB_TOKENS = 32;   // tokens per block when there are enough of them to fill the chip several times over
constexpr int DB_TOKENS_FEW = 8;   // otherwise: more, shorter blocks (4096 x 512 fp32 tokens: 10.5 against 22 us)
template <typename T, int EB>
__global__ __launch_bounds__(256) void dispatch_bwd_gate_kernel(const T *__restrict__ dxd,
                                                                const int32_t *__restrict__ row, int S, int M, int k,
                                                                const float *__restrict__ dlogits,
                                                                const float *__restrict__ wg, int E,
                                                                T *__restrict__ dx, int db_tokens) {
    const int m = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (m >= M) return;
    float w[EB][4];
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        const float4 v = e < E ? *reinterpret_cast<const float4 *>(wg + (size_t)e * M + m) : make_float4(0.f, 0.f, 0.f, 0.f);
        w[e][0] = v.x; w[e][1] = v.y; w[e][2] = v.z; w[e][3] = v.w;
    }
    const int i0 = blockIdx.x * db_tokens, i1 = min(i0 + db_tokens, S);
    // Eight tokens per batch; the first choice's row gathers of the next batch are in flight while the
    // current batch is finished: one token at a time, or one batch at a time, runs at the memory latency.
    constexpr int U = 8;
    typedef typename std::conditional<sizeof(T) == 2, uint2, float4>::type Raw;
    // (every load is issued unconditionally from a clamped address; what must not count - a token past the
    // block's end, a dropped pair - is masked when it is added: loads under a condition are waited for one by one)
    auto gather = [&](Raw (&v)[U], uint32_t (&ok)[U], int ib, int j) __attribute__((always_inline)) {
        int r[U];
#pragma unroll
        for (int u = 0; u < U; ++u) r[u] = row[(size_t)j * S + min(ib + u, i1 - 1)];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            ok[u] = (ib + u < i1 && r[u] >= 0) ? 0xffffffffu : 0u;
            v[u] = *reinterpret_cast<const Raw *>(dxd + (size_t)(r[u] & (int)ok[u]) * M + m);
        }
    };
    auto add = [&](float (&acc)[U][4], const Raw (&v)[U], const uint32_t (&ok)[U]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if constexpr (sizeof(T) == 2) {
                const uint32_t x = v[u].x & ok[u], y = v[u].y & ok[u];
                acc[u][0] += __uint_as_float(x << 16); acc[u][1] += __uint_as_float(x & 0xffff0000u);
                acc[u][2] += __uint_as_float(y << 16); acc[u][3] += __uint_as_float(y & 0xffff0000u);
            } else {
                acc[u][0] += __uint_as_float(__float_as_uint(v[u].x) & ok[u]);
                acc[u][1] += __uint_as_float(__float_as_uint(v[u].y) & ok[u]);
                acc[u][2] += __uint_as_float(__float_as_uint(v[u].z) & ok[u]);
                acc[u][3] += __uint_as_float(__float_as_uint(v[u].w) & ok[u]);
            }
        }
    };
    auto finish = [&](const Raw (&first)[U], const uint32_t (&first_ok)[U], int ib) __attribute__((always_inline)) {
        float acc[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u) acc[u][0] = acc[u][1] = acc[u][2] = acc[u][3] = 0.f;
        add(acc, first, first_ok);
        for (int j = 1; j < k; ++j) {
            Raw v[U];
            uint32_t ok[U];
            gather(v, ok, ib, j);
            add(acc, v, ok);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = ib + u;
            if (i >= i1) break;
            const float *dl = dlogits + (size_t)i * E;
#pragma unroll
            for (int e = 0; e < EB; ++e) {
                const float d = e < E ? dl[e] : 0.f;
#pragma unroll
                for (int q = 0; q < 4; ++q) acc[u][q] += d * w[e][q];
            }
            if constexpr (sizeof(T) == 2) {
                const bf16_t b0 = (bf16_t)acc[u][0], b1 = (bf16_t)acc[u][1], b2 = (bf16_t)acc[u][2], b3 = (bf16_t)acc[u][3];
                uint2 o;
                o.x = (uint32_t)__builtin_bit_cast(uint16_t, b0) | ((uint32_t)__builtin_bit_cast(uint16_t, b1) << 16);
                o.y = (uint32_t)__builtin_bit_cast(uint16_t, b2) | ((uint32_t)__builtin_bit_cast(uint16_t, b3) << 16);
                *reinterpret_cast<uint2 *>(dx + (size_t)i * M + m) = o;
            } else {
                *reinterpret_cast<float4 *>(dx + (size_t)i * M + m) = make_float4(acc[u][0], acc[u][1], acc[u][2], acc[u][3]);
            }
        }
    };
    Raw va[U], vb[U];
    uint32_t oka[U], okb[U];
    gather(va, oka, i0, 0);
    for (int ib = i0; ib < i1; ib += 2 * U) {
        gather(vb, okb, ib + U, 0);
        finish(va, oka, ib);
        gather(va, oka, ib + 2 * U, 0);
        if (ib + U < i1) finish(vb, okb, ib + U);
    }
}

// The same for bf16 tokens with the gate product on the matrix cores.  dlogits . Wg is a [tokens x E] by
// [E x M] product with E <= 32: one v_mfma_f32_16x16x32_bf16 per 16 tokens x 16 columns, both operands rounded
// to bf16 (the sum is rounded to bf16 on the way out anyway).  The fp32 kernel above spends 2 E VALU
// instructions per pair of output elements on it, which is what bounds it; here the VALU work is the
// unpack / add / pack of a copy.
// A block of eight waves covers 1024 columns, a wave 128 columns of 16 tokens at a time: its 8 product tiles go
// through an 8 KB LDS buffer of its own (the MFMA result has a lane hold four columns of one token; the
// row-major side wants eight columns of one token per lane), then every lane gathers 8 columns of one token's k
// source rows, adds and stores 16 bytes.  The first-choice gathers and the gradients of a group of tokens are issued one
// group ahead (two groups ahead: 14.7 against 14.3 us; all four groups' up front: 16.1, the weights' loads queue behind them).
constexpr int DM_TOKENS = 64;                 // tokens per block: four groups of 16 (32: +5 %, 16: +20 % at 16384 x 1024)
constexpr int DM_COLS = 128;                  // columns per wave
constexpr int DM_ROW = DM_COLS + 4;           // floats per token row of the LDS buffer: 4 rows apart = 16 banks apart
typedef __bf16 perm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float perm_f32x4 __attribute__((ext_vector_type(4)));
template <bool E8>   // E8: E is a multiple of 8, a lane's 8 gradients are two 16-byte loads
__global__ __launch_bounds__(512) void dispatch_bwd_gate_mfma_kernel(const bf16_t *__restrict__ dxd,
                                                                     const int32_t *__restrict__ row, int S, int M, int k,
                                                                     const float *__restrict__ dlogits,
                                                                     const float *__restrict__ wg, int E,
                                                                     bf16_t *__restrict__ dx) {
    __shared__ __align__(16) float s_t[8][16 * DM_ROW];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int col0 = (blockIdx.y * 8 + wave) * DM_COLS;      // this wave's first column
    if (col0 >= M) return;                                   // M is a multiple of 128: whole waves drop out
    float *buf = s_t[wave];
    const int tsel = lane >> 4, c8 = (lane & 15) * 8;        // row-major side: token within a quartet, first of 8 columns
    // the first-choice source rows of the 4 tokens this lane finishes in a group (tokens tok0 + 4 u + tsel)
    // (loads are unconditional, from clamped addresses, and what must not count is masked where it is used: a
    // load under a condition would make the compiler wait for all loads in flight at every such place)
    // (the first-choice rows of the block's 64 tokens come with one load, lane l holding token l's, and are handed
    // round between lanes: the gathers' addresses then wait for no load of their own)
    static_assert(DM_TOKENS == WAVE, "one first-choice row per lane");
    const int my_row = row[min((int)blockIdx.x * DM_TOKENS + lane, S - 1)];
    auto gather = [&](uint4 (&v)[4], uint32_t (&ok)[4], int tok0) __attribute__((always_inline)) {
        int r[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) r[u] = __shfl(my_row, (tok0 - (int)blockIdx.x * DM_TOKENS + 4 * u + tsel) & (WAVE - 1), WAVE);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            ok[u] = (tok0 + 4 * u + tsel < S && r[u] >= 0) ? 0xffffffffu : 0u;
            v[u] = *reinterpret_cast<const uint4 *>(dxd + (size_t)(r[u] & (int)ok[u]) * M + col0 + c8);
        }
    };
    uint4 src[4];
    uint32_t src_ok[4];
    gather(src, src_ok, blockIdx.x * DM_TOKENS);
    // A fragment of a group of 16 tokens: dlogits[tok0 + r16][8 kq .. 8 kq + 7], fetched one group ahead like the rows
    // (fetched where it is used, the product waited for it in every group: 15.0 -> 14.2 us at 16384 x 1024)
    auto load_d = [&](float (&d)[8], int tok0) __attribute__((always_inline)) {
        if constexpr (E8) {
            const float4 *dp = reinterpret_cast<const float4 *>(dlogits + (size_t)min(tok0 + r16, S - 1) * E + min(8 * kq, E - 8));
            const float4 d0 = dp[0], d1 = dp[1];
            d[0] = d0.x; d[1] = d0.y; d[2] = d0.z; d[3] = d0.w;
            d[4] = d1.x; d[5] = d1.y; d[6] = d1.z; d[7] = d1.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) d[i] = dlogits[(size_t)min(tok0 + r16, S - 1) * E + min(8 * kq + i, E - 1)];
        }
    };
    float d[8];
    load_d(d, blockIdx.x * DM_TOKENS);
    // B fragments: Wg[8 kq + i][col0 + 16 cb + r16], i = 0..7, for the wave's 8 column blocks.  Fetched row by row
    // with 16-byte loads (a lane takes 4 columns of the 8 experts of one group) and turned by way of the LDS
    // buffer, [expert group][column] with a group's 8 experts as one bf16x8 entry: picking them out of global
    // memory one float at a time took longer than the rest of the kernel.  Two expert groups per pass.
    perm_bf16x8 bfrag[8];
    {
        perm_bf16x8 *wt = reinterpret_cast<perm_bf16x8 *>(buf);      // [2][DM_COLS]
        const int c4 = (lane & 31) * 4, half = lane >> 5;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            if (pass * 16 >= E) break;
            const int eg = 2 * pass + half;
            float4 w[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) w[i] = *reinterpret_cast<const float4 *>(wg + (size_t)min(8 * eg + i, E - 1) * M + col0 + c4);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (8 * eg + i >= E) w[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            perm_bf16x8 *dst = wt + half * DM_COLS + c4;
            dst[0] = perm_bf16x8{(bf16_t)w[0].x, (bf16_t)w[1].x, (bf16_t)w[2].x, (bf16_t)w[3].x,
                                 (bf16_t)w[4].x, (bf16_t)w[5].x, (bf16_t)w[6].x, (bf16_t)w[7].x};
            dst[1] = perm_bf16x8{(bf16_t)w[0].y, (bf16_t)w[1].y, (bf16_t)w[2].y, (bf16_t)w[3].y,
                                 (bf16_t)w[4].y, (bf16_t)w[5].y, (bf16_t)w[6].y, (bf16_t)w[7].y};
            dst[2] = perm_bf16x8{(bf16_t)w[0].z, (bf16_t)w[1].z, (bf16_t)w[2].z, (bf16_t)w[3].z,
                                 (bf16_t)w[4].z, (bf16_t)w[5].z, (bf16_t)w[6].z, (bf16_t)w[7].z};
            dst[3] = perm_bf16x8{(bf16_t)w[0].w, (bf16_t)w[1].w, (bf16_t)w[2].w, (bf16_t)w[3].w,
                                 (bf16_t)w[4].w, (bf16_t)w[5].w, (bf16_t)w[6].w, (bf16_t)w[7].w};
            // the lanes whose expert group (kq) this pass staged pick up their fragments
            if ((kq >> 1) == pass) {
#pragma unroll
                for (int cb = 0; cb < 8; ++cb) bfrag[cb] = wt[(kq & 1) * DM_COLS + 16 * cb + r16];
            }
        }
        if (8 * kq >= E) {        // expert groups past the gate's size contribute nothing
            const bf16_t z = (bf16_t)0.0f;
#pragma unroll
            for (int cb = 0; cb < 8; ++cb) bfrag[cb] = perm_bf16x8{z, z, z, z, z, z, z, z};
        }
    }
#pragma unroll
    for (int g0 = 0; g0 < DM_TOKENS; g0 += 16) {
        const int tok0 = blockIdx.x * DM_TOKENS + g0;
        uint4 nxt[4];
        uint32_t nxt_ok[4];
        float d_nxt[8];
        if (g0 + 16 < DM_TOKENS) {
            gather(nxt, nxt_ok, tok0 + 16);
            load_d(d_nxt, tok0 + 16);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (tok0 + r16 >= S || 8 * kq + i >= E) d[i] = 0.f;
        const perm_bf16x8 afrag = {(bf16_t)d[0], (bf16_t)d[1], (bf16_t)d[2], (bf16_t)d[3],
                                   (bf16_t)d[4], (bf16_t)d[5], (bf16_t)d[6], (bf16_t)d[7]};
        // product tiles into LDS.  The gate's weights go into the first operand slot, so the four results of a lane
        // are four consecutive columns of one token (acc[r] = column 16 cb + 4 kq + r of token r16) and leave with
        // one 16-byte LDS write (a quarter wave's 16 rows are 16 banks-of-four apart: see DM_ROW)
#pragma unroll
        for (int cb = 0; cb < 8; ++cb) {
            const perm_f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfrag[cb], afrag, perm_f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            *reinterpret_cast<perm_f32x4 *>(buf + r16 * DM_ROW + 16 * cb + 4 * kq) = acc;
        }
        // (a wave's LDS buffer is written and read by that wave only: program order is enough)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int tl = 4 * u + tsel, t = tok0 + tl;
            const float4 p0 = *reinterpret_cast<const float4 *>(buf + tl * DM_ROW + c8);
            const float4 p1 = *reinterpret_cast<const float4 *>(buf + tl * DM_ROW + c8 + 4);
            float acc[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
            Vec<bf16_t> v;
            float f[8];
            v.raw = src[u];
            v.mask(src_ok[u]);
            v.unpack(f);
#pragma unroll
            for (int q = 0; q < 8; ++q) acc[q] += f[q];
            for (int j = 1; j < k; ++j) {
                const int r = row[(size_t)j * S + min(t, S - 1)];
                const uint32_t ok = (t < S && r >= 0) ? 0xffffffffu : 0u;
                v.load(dxd + (size_t)(r & (int)ok) * M + col0 + c8);
                v.mask(ok);
                v.unpack(f);
#pragma unroll
                for (int q = 0; q < 8; ++q) acc[q] += f[q];
            }
            if (t < S) {
                v.pack(acc);
                v.store(dx + (size_t)t * M + col0 + c8);
            }
        }
        if (g0 + 16 < DM_TOKENS) {
#pragma unroll
            for (int u = 0; u < 4; ++u) { src[u] = nxt[u]; src_ok[u] = nxt_ok[u]; }
#pragma unroll
            for (int i = 0; i < 8; ++i) d[i] = d_nxt[i];
        }
    }
}

// Gate weight gradient dWg[e, m] = sum_i dlogits[i, e] * x[i, m] (the Linear backward that
// autograd runs for MOLETopk, MOLE/utils/Ugate.py:12), in two deterministic passes: blocks of
// GW_TOKENS tokens write partial [E, M] sums, a second kernel adds the partials in order.
constexpr int GW_TOKENS = 64;
template <typename T, int EB>
__global__ __launch_bounds__(256) void gate_wgrad_partial_kernel(const float *__restrict__ dlogits,
                                                                 const T *__restrict__ x, int S, int E, int M,
                                                                 float *__restrict__ part) {
    __shared__ __align__(16) float s_dl[GW_TOKENS][EB];
    const int i0 = blockIdx.x * GW_TOKENS;
    const int nt = min(GW_TOKENS, S - i0);
    for (int idx = threadIdx.x; idx < GW_TOKENS * EB; idx += 256) {
        const int t = idx / EB, e = idx % EB;
        s_dl[t][e] = (t < nt && e < E) ? dlogits[(size_t)(i0 + t) * E + e] : 0.f;
    }
    __syncthreads();
    const int m = (blockIdx.y * 256 + threadIdx.x) * 2;    // two columns per thread
    if (m >= M) return;
    float acc[EB][2];
#pragma unroll
    for (int e = 0; e < EB; ++e) acc[e][0] = acc[e][1] = 0.f;
    const T *px = x + (size_t)i0 * M + m;
    // eight rows per batch, the next batch's loads in flight while the current one is used
    auto load8 = [&](float (&xv)[8][2], int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = min(t0 + u, nt - 1);
            if constexpr (sizeof(T) == 2) {
                const uint32_t v = *reinterpret_cast<const uint32_t *>(px + (size_t)t * M);
                xv[u][0] = __uint_as_float(v << 16); xv[u][1] = __uint_as_float(v & 0xffff0000u);
            } else {
                const float2 v = *reinterpret_cast<const float2 *>(px + (size_t)t * M);
                xv[u][0] = v.x; xv[u][1] = v.y;
            }
        }
    };
    auto use8 = [&](const float (&xv)[8][2], int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (t0 + u >= nt) break;
#pragma unroll
            for (int e = 0; e < EB; e += 4) {
                const float4 d = *reinterpret_cast<const float4 *>(&s_dl[t0 + u][e]);   // same address in every lane
                acc[e][0] += d.x * xv[u][0]; acc[e][1] += d.x * xv[u][1];
                acc[e + 1][0] += d.y * xv[u][0]; acc[e + 1][1] += d.y * xv[u][1];
                acc[e + 2][0] += d.z * xv[u][0]; acc[e + 2][1] += d.z * xv[u][1];
                acc[e + 3][0] += d.w * xv[u][0]; acc[e + 3][1] += d.w * xv[u][1];
            }
        }
    };
    float xa[8][2], xb[8][2];
    load8(xa, 0);
    for (int t0 = 0; t0 < nt; t0 += 16) {
        load8(xb, t0 + 8);
        use8(xa, t0);
        load8(xa, t0 + 16);
        use8(xb, t0 + 8);
    }
#pragma unroll
    for (int e = 0; e < EB; ++e)
        if (e < E)
            *reinterpret_cast<float2 *>(part + ((size_t)blockIdx.x * E + e) * M + m) = make_float2(acc[e][0], acc[e][1]);
}
// The partial sums on the matrix cores, for bf16 tokens and gates of up to 256 experts:
// part[chunk][e][m] = sum over the chunk's tokens of dlogits[t][e] x[t][m], a [E x tokens] by [tokens x M]
// product per chunk with v_mfma_f32_16x16x32_bf16 and fp32 accumulation.  dlogits is fp32: it enters as the sum
// of two bf16 numbers (the rounded value and the rounded remainder, 16 significant bits together), each
// multiplied separately, so the result stays as close to the exact sum as the fp32 accumulation allows.
// A block of four waves takes one chunk of tokens, 256 columns (64 per wave) and up to 64 experts (grid z walks
// the rest).  The contraction runs over tokens, along which neither operand is contiguous in memory, so both
// are turned in LDS: they are staged as they lie in memory, [token][expert] for the chunk's dlogits (128 tokens
// at a time, shared by the block) and [token][column] for x (32 tokens at a time per wave), and read back with
// the transposing ds_read_b64_tr_b16 (a group of 16 lanes receives a 4-token x 16-column block column by column).  The next
// 128 tokens' rows of x and dlogits are in flight while the current ones are multiplied.
constexpr int GM_KSTEP = 32;                  // tokens per MFMA
constexpr int GM_XROW = 72;                   // bf16 per token row of a wave's x tile: 64 columns + 16 bytes,
                                              // so that the 4 rows of a transposing read fall into distinct banks
constexpr int GM_SUB = 128;                   // tokens whose dlogits are staged at a time
typedef short perm_s16x4 __attribute__((ext_vector_type(4)));
template <int EG, bool DL4>   // groups of 16 experts per block; DL4: E is a multiple of 4, dlogits come by 16-byte loads
__global__ __launch_bounds__(256, 2) void gate_wgrad_mfma_kernel(const float *__restrict__ dlogits,
                                                              const bf16_t *__restrict__ x, int S, int E, int M,
                                                              int chunk, int nchunks, int nz, float *__restrict__ part) {
    // staged dlogits, [token][expert] like x: rounded values and rounded remainders.  Row length: the group's
    // experts + padding that puts the 4 token rows of a transposing read into distinct banks
    constexpr int DLROW = 16 * EG + (EG == 2 ? 16 : 8);
    __shared__ __align__(16) bf16_t s_dl[2][GM_SUB * DLROW];
    __shared__ __align__(16) bf16_t s_x[4 * GM_KSTEP * GM_XROW];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    // block -> (chunk, column block, expert group).  Blocks go round-robin to the 8 XCDs; the nz expert groups of
    // one (chunk, column block) unit take consecutive slots of one XCD, so the unit's x tile comes out of that
    // XCD's L2 for all but the first of them.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int unit = (slot / nz) * 8 + xcd, zi = slot % nz;
    if (unit >= nchunks * ((M + 255) / 256)) return;     // padding blocks of the last round of units
    const int ci = unit % nchunks, yi = unit / nchunks;
    const int tok0 = ci * chunk, ntok = min(chunk, S - tok0);
    const int e0 = zi * 16 * EG;
    const int col0 = yi * 256 + wave * 64;
    const bool active = col0 < M;             // M is a multiple of 64: a wave is in or out as a whole
    bf16_t *xt = s_x + wave * (GM_KSTEP * GM_XROW);
    perm_f32x4 acc[EG][4];
#pragma unroll
    for (int g = 0; g < EG; ++g)
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) acc[g][cb] = perm_f32x4{0.f, 0.f, 0.f, 0.f};
    // a wave's x tile of one step: 32 tokens x 64 columns = 4 loads of 16 bytes per lane (token 8 i + lane / 8)
    // Every load is issued unconditionally from a clamped, valid address, and what lies past the chunk is
    // replaced by zero only where the value is used, a sub-chunk later: a load under a branch, or one whose
    // value is touched right away, makes the compiler wait for all outstanding loads, which undoes the prefetch.
    const int lt = lane >> 3, lc = (lane & 7) * 8;
    const bf16_t *xcol = x + (active ? col0 : 0) + lc;
    auto fetch = [&](uint4 (&v)[4], int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = k0 + 8 * i + lt;
            v[i] = *reinterpret_cast<const uint4 *>(xcol + (size_t)(tok0 + min(t, ntok - 1)) * M);
        }
    };
    // a thread's share of the dlogits of GM_SUB tokens: expert de of the block's group (expert fastest across
    // threads: the global reads are whole rows of dlogits), tokens dt0, dt0 + DL_TSTEP, ...; fetched into
    // registers one sub-chunk ahead, so the loads are in flight while the current sub-chunk is multiplied
    // (DL4: four consecutive experts per thread and load, a quarter of the load instructions)
    constexpr int DL_V = DL4 ? 4 : 1;
    constexpr int DL_W = 16 * EG / DL_V, DL_N = GM_SUB * DL_W / 256, DL_TSTEP = 256 / DL_W;
    const int de = (threadIdx.x % DL_W) * DL_V, dt0 = threadIdx.x / DL_W;
    float dl[DL_N][DL_V];
    const bool dl_in = e0 + de < E;
    const float *dl_col = dlogits + min(e0 + de, E - DL_V);
    auto fetch_dl = [&](int sub0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < DL_N; ++i) {
            const int t = sub0 + dt0 + DL_TSTEP * i;
            const float *p = dl_col + (size_t)(tok0 + min(t, ntok - 1)) * E;
            if constexpr (DL4) {
                const float4 v = *reinterpret_cast<const float4 *>(p);
                dl[i][0] = v.x; dl[i][1] = v.y; dl[i][2] = v.z; dl[i][3] = v.w;
            } else {
                dl[i][0] = *p;
            }
        }
    };
    // the x tiles of a whole sub-chunk (GM_SUB / GM_KSTEP = 4 steps) are in flight at any time: a step's
    // registers are refilled with the same step of the next sub-chunk as soon as its tile is in LDS
    constexpr int NQ = GM_SUB / GM_KSTEP;
    uint4 q[NQ][4];
#pragma unroll
    for (int i = 0; i < NQ; ++i) fetch(q[i], GM_KSTEP * i);
    fetch_dl(0);
    for (int sub0 = 0; sub0 < ntok; sub0 += GM_SUB) {
        // this sub-chunk's dlogits -> LDS, transposed and split into rounded value and rounded remainder
        __syncthreads();
#pragma unroll
        for (int i = 0; i < DL_N; ++i) {
            const int t = dt0 + DL_TSTEP * i;
#pragma unroll
            for (int c = 0; c < DL_V; ++c) {
                const float v = (sub0 + t < ntok && dl_in) ? dl[i][c] : 0.f;
                const bf16_t hi = (bf16_t)v;
                s_dl[0][t * DLROW + de + c] = hi;
                s_dl[1][t * DLROW + de + c] = (bf16_t)(v - (float)hi);
            }
        }
        __syncthreads();
        fetch_dl(sub0 + GM_SUB);              // past the chunk's end: zeros
#pragma unroll
        for (int qi = 0; qi < NQ; ++qi) {       // steps past the chunk's end multiply zeros
            const int k0 = sub0 + GM_KSTEP * qi;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *reinterpret_cast<uint4 *>(xt + (8 * i + lt) * GM_XROW + lc) =
                    k0 + 8 * i + lt < ntok ? q[qi][i] : make_uint4(0, 0, 0, 0);
            // (the tile is written and read by this wave only: program order is enough)
            fetch(q[qi], k0 + GM_SUB);        // past the chunk's end: zeros
            // a fragment by two transposing reads: 4 + 4 tokens from 8 kq + (r16 >> 2) on, 16 columns from col on,
            // 4 (r16 & 3) .. per lane; lane r16 receives column col + r16 of the 8 tokens 8 kq ..
            auto frag = [&](const bf16_t *tile, int row_len, int col) __attribute__((always_inline)) {
                const bf16_t *p = tile + (8 * kq + (r16 >> 2)) * row_len + col + 4 * (r16 & 3);
                const perm_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((perm_s16x4 __attribute__((address_space(3))) *)(p));
                const perm_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((perm_s16x4 __attribute__((address_space(3))) *)(p + 4 * row_len));
                typedef short s16x8 __attribute__((ext_vector_type(8)));
                const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                return __builtin_bit_cast(perm_bf16x8, v);
            };
            perm_bf16x8 a[EG], al[EG];
#pragma unroll
            for (int g = 0; g < EG; ++g) {
                a[g] = frag(s_dl[0] + (k0 - sub0) * DLROW, DLROW, 16 * g);
                al[g] = frag(s_dl[1] + (k0 - sub0) * DLROW, DLROW, 16 * g);
            }
#pragma unroll
            for (int cb = 0; cb < 4; ++cb) {
                const perm_bf16x8 b = frag(xt, GM_XROW, 16 * cb);
#pragma unroll
                for (int g = 0; g < EG; ++g) {
                    acc[g][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[g], b, acc[g][cb], 0, 0, 0);
                    acc[g][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[g], b, acc[g][cb], 0, 0, 0);
                }
            }
        }
    }
    if (!active) return;
    // acc[g][cb][r] = expert e0 + 16 g + 4 kq + r, column col0 + 16 cb + r16
    float *out = part + (size_t)ci * E * M;
#pragma unroll
    for (int g = 0; g < EG; ++g)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int e = e0 + 16 * g + 4 * kq + r;
            if (e >= E) continue;
#pragma unroll
            for (int cb = 0; cb < 4; ++cb) out[(size_t)e * M + col0 + 16 * cb + r16] = acc[g][cb][r];
        }
}

// tokens per chunk of the kernel above: chunks of 128 tokens while the partials stay within 32 MB (or 8
// chunks), twice as long as often as needed beyond
static int gate_wgrad_mfma_chunk(int S, int E, int M) {
    const size_t per_chunk = (size_t)E * M * sizeof(float);
    size_t max_chunks = (32u << 20) / per_chunk;
    if (max_chunks < 8) max_chunks = 8;
    int chunk = 128;
    while ((size_t)ceil_div(S, chunk) > max_chunks && chunk < (1 << 24)) chunk *= 2;
    return chunk;
}
static bool gate_wgrad_mfma_ok(int dtype, int S, int E, int M) {
    return dtype == MOLE_BF16 && E <= 256 && M % 64 == 0 && S > 0 &&
           (size_t)ceil_div(S, gate_wgrad_mfma_chunk(S, E, M)) <= 65535;
}

// sums the partials in a fixed order: 16 slices of the block list per group of four outputs, then the
// slices in order
__global__ __launch_bounds__(256) void gate_wgrad_reduce_kernel(const float *__restrict__ part, int nblocks, int EM,
                                                                float *__restrict__ dwg) {
    __shared__ float4 s_acc[16][16];
    const int o = threadIdx.x & 15, slice = threadIdx.x >> 4;
    const int idx = (blockIdx.x * 16 + o) * 4;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (nblocks > 0) {
        // eight partials per batch, loaded unconditionally from clamped addresses so that they are in flight
        // together, and added in order; what lies past the slice is cleared by a bit mask
        const int per = (nblocks + 15) / 16;
        const int b1 = min(nblocks, (slice + 1) * per);
        const float *src = part + (idx < EM ? idx : 0);
        for (int b0 = slice * per; b0 < b1; b0 += 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const float4 *>(src + (size_t)min(b0 + u, nblocks - 1) * EM);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t keep = b0 + u < b1 ? 0xffffffffu : 0u;
                acc.x += __uint_as_float(__float_as_uint(v[u].x) & keep);
                acc.y += __uint_as_float(__float_as_uint(v[u].y) & keep);
                acc.z += __uint_as_float(__float_as_uint(v[u].z) & keep);
                acc.w += __uint_as_float(__float_as_uint(v[u].w) & keep);
            }
        }
    }
    s_acc[slice][o] = acc;
    __syncthreads();
    if (slice == 0 && idx < EM) {
        float4 r = s_acc[0][o];
#pragma unroll
        for (int sl = 1; sl < 16; ++sl) { r.x += s_acc[sl][o].x; r.y += s_acc[sl][o].y; r.z += s_acc[sl][o].z; r.w += s_acc[sl][o].w; }
        *reinterpret_cast<float4 *>(dwg + idx) = r;
    }
}

template <typename T, int K, int TPW>
__global__ __launch_bounds__(PM_THREADS) void combine_fwd_kernel(const T *__restrict__ o,
                                                                 const int32_t *__restrict__ row,
                                                                 const float *__restrict__ gates, int S, int M,
                                                                 int k, T *__restrict__ y) {
    const int i0 = (blockIdx.x * (PM_THREADS / WAVE) + (threadIdx.x >> 6)) * TPW;
    if (i0 >= S) return;
    const int lane = lane_id();
    int r[TPW][K];
    uint32_t keep[TPW][K];
    float g[TPW][K];
    load_rows_multi<K, TPW>(row, S, k, i0, r, keep);
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int j = 0; j < K; ++j) g[t][j] = gates[(size_t)min(j, k - 1) * S + min(i0 + t, S - 1)];
    constexpr int N = Vec<T>::N;
    constexpr int U = K >= 16 ? 1 : PM_U;
    const int chunks = M / N;
    for (int c0 = lane; c0 < chunks; c0 += U * WAVE) {
        Vec<T> v[TPW][U][K];
#pragma unroll
        for (int t = 0; t < TPW; ++t)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * WAVE;
                const size_t off = (size_t)(c < chunks ? c : c0) * N;
#pragma unroll
                for (int j = 0; j < K; ++j) v[t][u][j].load(o + (size_t)r[t][j] * M + off);
            }
#pragma unroll
        for (int t = 0; t < TPW; ++t)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * WAVE;
                if (c >= chunks || i0 + t >= S) continue;
                float acc[N], f[N];
#pragma unroll
                for (int q = 0; q < N; ++q) acc[q] = 0.f;
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    v[t][u][j].mask(keep[t][j]);         // a slot that does not count contributes g * (+0)
                    v[t][u][j].unpack(f);
                    const float gj = __uint_as_float(__float_as_uint(g[t][j]) & keep[t][j]);
#pragma unroll
                    for (int q = 0; q < N; ++q) acc[q] += gj * f[q];
                }
                Vec<T> out;
                out.pack(acc);
                out.store(y + (size_t)(i0 + t) * M + (size_t)c * N);
            }
    }
}

// The row streaming of the combine backward for token i: d_o[row_j] = g_j dy[i], and the k dot products <dy[i], o[row_j]>
// summed over the wave (every lane ends up with all of them).
template <typename T, int K>
__device__ __forceinline__ void combine_bwd_rows(const T *__restrict__ dy, const T *__restrict__ o,
                                                 const int32_t *__restrict__ row, const float *__restrict__ gates, int S,
                                                 int M, int k, int i, T *__restrict__ d_o, float (&dot)[K]) {
    const int lane = lane_id();
    int r[K];
    uint32_t keep[K];
    float g[K];
    load_rows<K>(row, S, k, i, r, keep);
#pragma unroll
    for (int j = 0; j < K; ++j) {
        g[j] = gates[(size_t)min(j, k - 1) * S + i];
        dot[j] = 0.f;
    }
    constexpr int N = Vec<T>::N;
    constexpr int U = K >= 8 ? 1 : PM_U;
    const int chunks = M / N;
    for (int c0 = lane; c0 < chunks; c0 += U * WAVE) {
        Vec<T> a[U], b[U][K];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + u * WAVE;
            const size_t off = (size_t)(c < chunks ? c : c0) * N;
            // dy and the experts' outputs are read here for the last time, while the d_o written below is an operand
            // of the two products that follow: streaming loads leave the caches to d_o (16384 x 1024 bf16: the
            // weight gradient and the GELU' product after this kernel each 2 us shorter, this kernel unchanged)
            a[u].load_nt(dy + (size_t)i * M + off);
#pragma unroll
            for (int j = 0; j < K; ++j) b[u][j].load_nt(o + (size_t)r[j] * M + off);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + u * WAVE;
            if (c >= chunks) continue;
            float fa[N];
            a[u].unpack(fa);
#pragma unroll
            for (int j = 0; j < K; ++j) {
                float fb[N], fo[N];
                b[u][j].mask(keep[j]);         // a slot that does not count: dot stays 0, nothing is stored
                b[u][j].unpack(fb);
#pragma unroll
                for (int q = 0; q < N; ++q) {
                    dot[j] += fa[q] * fb[q];
                    fo[q] = g[j] * fa[q];
                }
                if (keep[j]) {
                    Vec<T> w;
                    w.pack(fo);
                    w.store(d_o + (size_t)r[j] * M + (size_t)c * N);
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < K; ++j) dot[j] = wave_sum(dot[j]);
}

template <typename T, int K>
__global__ __launch_bounds__(PM_THREADS) void combine_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ o,
                                                                 const int32_t *__restrict__ row,
                                                                 const float *__restrict__ gates, int S, int M,
                                                                 int k, T *__restrict__ d_o,
                                                                 float *__restrict__ dgates) {
    const int i = blockIdx.x * (PM_THREADS / WAVE) + (threadIdx.x >> 6);
    if (i >= S) return;
    float dot[K];
    combine_bwd_rows<T, K>(dy, o, row, gates, S, M, k, i, d_o, dot);
#pragma unroll
    for (int j = 0; j < K; ++j)
        if (lane_id() == 0 && j < k) dgates[(size_t)j * S + i] = dot[j];
}

// The combine backward with the gate's backward in its tail: the k gate gradients of a token never leave the wave
// that formed them.  From them: the gradient of the raw gate values through the normalisation gate_j = graw_j /
// max(sum graw, eps), scattered to the chosen experts' scores, plus the load-balancing loss's term when counts0 and
// d_l_aux are given, then through the softmax.  Lane l holds experts l, l + 64, ... (VPL of them); the token's score
// row and indices are requested before the rows are streamed, so the tail waits for no memory.
struct GateBwdArgs {
    const float *scores;      // [S,E]
    const int32_t *idx;       // [k,S]
    int E, normalize, through_softmax;
    const int32_t *counts0;   // [E] or null
    const float *d_l_aux;     // [1] or null
    float *dlogits;           // [S,E]
};
template <typename T, int K, int VPL>
__global__ __launch_bounds__(PM_THREADS) void combine_bwd_gate_kernel(const T *__restrict__ dy, const T *__restrict__ o,
                                                                      const int32_t *__restrict__ row,
                                                                      const float *__restrict__ gates, int S, int M,
                                                                      int k, T *__restrict__ d_o, const GateBwdArgs ga) {
    const int i = blockIdx.x * (PM_THREADS / WAVE) + (threadIdx.x >> 6);
    if (i >= S) return;
    const int lane = lane_id(), E = ga.E;
    // the token's scores, the choice this lane looks after (lanes below k), and that choice's raw gate value
    float s[VPL], ds[VPL];
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = lane + 64 * r;
        s[r] = ga.scores[(size_t)i * E + min(e, E - 1)];
    }
    const int my_e = ga.idx[(size_t)min(lane, k - 1) * S + i];
    float dot[K];
    combine_bwd_rows<T, K>(dy, o, row, gates, S, M, k, i, d_o, dot);
    // the raw gate value of this lane's choice is the score of expert my_e, which lane my_e % 64 holds: handed over
    // between lanes (a load of it would have to wait for my_e first, one more memory latency per wave)
    float my_gr = 0.f;
    const int e_c = min(max(my_e, 0), E - 1);
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const float v = __shfl(s[r], e_c & 63, WAVE);
        if ((e_c >> 6) == r) my_gr = v;
    }
    float my_dg = 0.f;
#pragma unroll
    for (int j = 0; j < K; ++j)
        if (lane == j) my_dg = dot[j];
    if (lane >= k) { my_dg = 0.f; my_gr = 0.f; }
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        if (lane + 64 * r >= E) s[r] = 0.f;
        ds[r] = 0.f;
    }
    if (ga.counts0 != nullptr) {
        const float scale = ga.d_l_aux[0] * ((float)E / ((float)S * (float)S));
#pragma unroll
        for (int r = 0; r < VPL; ++r) ds[r] = scale * (float)ga.counts0[min(lane + 64 * r, E - 1)];
    }
    constexpr float EPS = 1.1920928955078125e-07f;
    const float denom = wave_sum(my_gr);
    const float dotg = wave_sum(my_dg * my_gr);
    const bool norm = k > 1 && ga.normalize;
    const bool clamped = denom < EPS;
    const float den = clamped ? EPS : denom;
    const float sub = (norm && !clamped) ? dotg / (den * den) : 0.f;
    const float my_dgraw = norm ? my_dg / den - sub : my_dg;
    for (int j = 0; j < k; ++j) {
        const int e = __builtin_amdgcn_readlane(my_e, j);
        const float dgraw = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_dgraw), j));
        if ((e & 63) == lane) {
            const int rr = e >> 6;
#pragma unroll
            for (int r = 0; r < VPL; ++r)
                if (r == rr) ds[r] += dgraw;
        }
    }
    float dsum = 0.f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) dsum += ds[r] * s[r];
    dsum = wave_sum(dsum);
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = lane + 64 * r;
        if (e < E) ga.dlogits[(size_t)i * E + e] = ga.through_softmax ? s[r] * (ds[r] - dsum) : ds[r];
    }
}

// rows offsets[e]+kept_rows[e] .. offsets[e+1] of expert e are padding: zero them
template <typename T>
__global__ __launch_bounds__(PM_THREADS) void zero_pad_rows_kernel(T *__restrict__ buf,
                                                                   const int32_t *__restrict__ kept_rows,
                                                                   const int32_t *__restrict__ offsets, int M) {
    const int e = blockIdx.y;
    const int lo = offsets[e] + kept_rows[e], hi = offsets[e + 1];
    const int lane = lane_id();
    constexpr int N = Vec<T>::N;
    const int chunks = M / N;
    Vec<T> z;
    z.zero();
    for (int r = lo + blockIdx.x * (PM_THREADS / WAVE) + (threadIdx.x >> 6); r < hi;
         r += gridDim.x * (PM_THREADS / WAVE))
        for (int c = lane; c < chunks; c += WAVE) z.store(buf + (size_t)r * M + (size_t)c * N);
}

static int check_perm(const char *fn, int dtype, int S, int M, int k) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "%s: bad dtype %d", fn, dtype);
    MOLE_REQUIRE(S >= 0 && M > 0 && k >= 1 && k <= MOLE_MAX_TOPK, "%s: bad sizes S=%d M=%d k=%d", fn, S, M, k);
    MOLE_REQUIRE(M % (dtype == MOLE_BF16 ? 8 : 4) == 0, "%s: M=%d must be a multiple of %d", fn, M,
                 dtype == MOLE_BF16 ? 8 : 4);
    return 0;
}
static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// The wave-per-token kernels for the smallest K in {1, 2, 4, 8, 16} that holds k.  The scatter and the gather take
// several tokens per wave when there is one choice per token (TPW1: 8 for the scatter, whose source rows follow one
// another in memory - 16 loads in flight; 4 for the gather - 8 in flight; measured at 16384 x 1024 bf16: 11.5 -> 9.0-9.7 us
// and 12.0 -> 11.3 us, slower again with more and, at two choices per token, with any), as long as that leaves two
// blocks for every CU.  The combine backward measured best with one token per wave (two: 19.2 against 18.8 us,
// four: 20.9) and keeps the one-token kernel.
static int perm_tpw(int S, int k, int tpw1) {
    int tpw = k <= 1 && tpw1 > 1 ? tpw1 : 1;
    while (tpw > 1 && ceil_div(S, (PM_THREADS / WAVE) * tpw) < 512) tpw >>= 1;
    return tpw;
}
#define PM_LAUNCH_KT(KID, KERNEL, T, TPW1, ...)                                                                   \
    do {                                                                                                         \
        const dim3 blk_(PM_THREADS);                                                                             \
        const int tpw_ = perm_tpw(S, k, TPW1);                                                                   \
        const dim3 grid_(ceil_div(S, (PM_THREADS / WAVE) * tpw_));                                               \
        if (k <= 1 && tpw_ == 8) timed_launch(KID, KERNEL<T, 1, (TPW1 >= 8 ? 8 : 1)>, grid_, blk_, 0, (hipStream_t)stream, __VA_ARGS__);   \
        else if (k <= 1 && tpw_ == 4) timed_launch(KID, KERNEL<T, 1, (TPW1 >= 4 ? 4 : 1)>, grid_, blk_, 0, (hipStream_t)stream, __VA_ARGS__); \
        else if (k <= 1 && tpw_ == 2) timed_launch(KID, KERNEL<T, 1, (TPW1 >= 2 ? 2 : 1)>, grid_, blk_, 0, (hipStream_t)stream, __VA_ARGS__); \
        else if (k <= 1) timed_launch(KID, KERNEL<T, 1, 1>, grid_, blk_, 0, (hipStream_t)stream, __VA_ARGS__);   \
        else if (k <= 2) timed_launch(KID, KERNEL<T, 2, 1>, grid_, blk_, 0, (hipStream_t)stream, __VA_ARGS__);   \
        else if (k <= 4) timed_launch(KID, KERNEL<T, 4, 1>, grid_, blk_, 0, (hipStream_t)stream, __VA_ARGS__);   \
        else if (k <= 8) timed_launch(KID, KERNEL<T, 8, 1>, grid_, blk_, 0, (hipStream_t)stream, __VA_ARGS__);   \
        else timed_launch(KID, KERNEL<T, 16, 1>, grid_, blk_, 0, (hipStream_t)stream, __VA_ARGS__);              \
    } while (0)
// one token per wave
#define PM_LAUNCH_K(KID, KERNEL, T, ...)                                                                         \
    do {                                                                                                         \
        const dim3 blk_(PM_THREADS);                                                                             \
        if (k <= 1) timed_launch(KID, KERNEL<T, 1>, grid, blk_, 0, (hipStream_t)stream, __VA_ARGS__);            \
        else if (k <= 2) timed_launch(KID, KERNEL<T, 2>, grid, blk_, 0, (hipStream_t)stream, __VA_ARGS__);       \
        else if (k <= 4) timed_launch(KID, KERNEL<T, 4>, grid, blk_, 0, (hipStream_t)stream, __VA_ARGS__);       \
        else if (k <= 8) timed_launch(KID, KERNEL<T, 8>, grid, blk_, 0, (hipStream_t)stream, __VA_ARGS__);       \
        else timed_launch(KID, KERNEL<T, 16>, grid, blk_, 0, (hipStream_t)stream, __VA_ARGS__);                  \
    } while (0)

}  // namespace mole

using namespace mole;

extern "C" int mole_dispatch_fwd(const void *x, int dtype, const int32_t *row, int S, int M, int k, void *xd,
                                 mole_stream_t stream) {
    if (int rc = check_perm("mole_dispatch_fwd", dtype, S, M, k)) return rc;
    if (S == 0) return 0;
    MOLE_REQUIRE(x && row && xd && aligned16(x) && aligned16(xd), "mole_dispatch_fwd: null or misaligned pointer");
    if (dtype == MOLE_BF16)
        PM_LAUNCH_KT(MOLE_K_DISPATCH_FWD, dispatch_fwd_kernel, bf16_t, 8, (const bf16_t *)x, row, S, M, k, (bf16_t *)xd);
    else
        PM_LAUNCH_KT(MOLE_K_DISPATCH_FWD, dispatch_fwd_kernel, float, 8, (const float *)x, row, S, M, k, (float *)xd);
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" int mole_dispatch_bwd(const void *dxd, int dtype, const int32_t *row, int S, int M, int k,
                                 const float *dlogits, const float *wg, int E, const void *dx_add, void *dx,
                                 mole_stream_t stream) {
    if (int rc = check_perm("mole_dispatch_bwd", dtype, S, M, k)) return rc;
    if (S == 0) return 0;
    MOLE_REQUIRE(dxd && row && dx && aligned16(dxd) && aligned16(dx), "mole_dispatch_bwd: null or misaligned pointer");
    MOLE_REQUIRE(dlogits == nullptr || (wg != nullptr && E >= 1 && aligned16(wg) && M % 4 == 0),
                 "mole_dispatch_bwd: dlogits given without a valid wg/E");
    MOLE_REQUIRE(dx_add == nullptr || aligned16(dx_add), "mole_dispatch_bwd: misaligned dx_add");
    if (dlogits != nullptr && dx_add == nullptr && E <= 32 && M % DM_COLS == 0 && dtype == MOLE_BF16) {
        const dim3 grid(ceil_div(S, DM_TOKENS), ceil_div(M, 8 * DM_COLS));
        if (E % 8 == 0 && ((uintptr_t)dlogits & 15) == 0)
            timed_launch(MOLE_K_DISPATCH_BWD, dispatch_bwd_gate_mfma_kernel<true>, grid, dim3(512), 0, (hipStream_t)stream,
                         (const bf16_t *)dxd, row, S, M, k, dlogits, wg, E, (bf16_t *)dx);
        else
            timed_launch(MOLE_K_DISPATCH_BWD, dispatch_bwd_gate_mfma_kernel<false>, grid, dim3(512), 0, (hipStream_t)stream,
                         (const bf16_t *)dxd, row, S, M, k, dlogits, wg, E, (bf16_t *)dx);
        MOLE_LAUNCH_CHECK();
        return 0;
    }
    if (dlogits != nullptr && dx_add == nullptr && E <= 32 && M % 4 == 0) {
        const int db_tokens = (long)ceil_div(S, DB_TOKENS) * ceil_div(M, 1024) < 1024 ? DB_TOKENS_FEW : DB_TOKENS;
        const dim3 grid(ceil_div(S, db_tokens), ceil_div(M, 1024));
        hipStream_t st = (hipStream_t)stream;
#define MOLE_DB(T, EB) timed_launch(MOLE_K_DISPATCH_BWD, dispatch_bwd_gate_kernel<T, EB>, grid, dim3(256), 0, st, (const T *)dxd, row, S, M, k, dlogits, wg, E, (T *)dx, db_tokens)
        if (dtype == MOLE_BF16) {
            if (E <= 8) MOLE_DB(bf16_t, 8); else if (E <= 16) MOLE_DB(bf16_t, 16); else MOLE_DB(bf16_t, 32);
        } else {
            if (E <= 8) MOLE_DB(float, 8); else if (E <= 16) MOLE_DB(float, 16); else MOLE_DB(float, 32);
        }
#undef MOLE_DB
        MOLE_LAUNCH_CHECK();
        return 0;
    }
    const dim3 grid(ceil_div(S, PM_THREADS / WAVE));
    if (dtype == MOLE_BF16)
        PM_LAUNCH_K(MOLE_K_DISPATCH_BWD, dispatch_bwd_kernel, bf16_t, (const bf16_t *)dxd, row, S, M, k, dlogits, wg, E, (const bf16_t *)dx_add, (bf16_t *)dx);
    else
        PM_LAUNCH_K(MOLE_K_DISPATCH_BWD, dispatch_bwd_kernel, float, (const float *)dxd, row, S, M, k, dlogits, wg, E, (const float *)dx_add, (float *)dx);
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" size_t mole_gate_wgrad_workspace_bytes(int S, int E, int M) {
    if (S <= 0 || E <= 0 || M <= 0) return 0;
    // enough for either kernel: the caller does not say the dtype here (small gates: the VALU kernel's 64-token
    // partials; large gates only run on the matrix cores, with their own chunking)
    const size_t mfma = (size_t)ceil_div(S, gate_wgrad_mfma_chunk(S, E, M)) * E * M * sizeof(float);
    const size_t valu = E <= 32 ? (size_t)ceil_div(S, GW_TOKENS) * E * M * sizeof(float) : 0;
    return mfma > valu ? mfma : valu;
}

extern "C" int mole_gate_wgrad(const float *dlogits, const void *x, int dtype, int S, int E, int M, float *dwg,
                               void *workspace, size_t workspace_bytes, mole_stream_t stream) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "mole_gate_wgrad: bad dtype %d", dtype);
    MOLE_REQUIRE(S >= 0 && E >= 1 && M > 0 && M % 4 == 0 && (E <= 32 || gate_wgrad_mfma_ok(dtype, S, E, M) || S == 0),
                 "mole_gate_wgrad: need E <= 32, or bf16 tokens with E <= 256 and M %% 64 == 0 (S=%d E=%d M=%d dtype=%d)", S, E, M, dtype);
    MOLE_REQUIRE(dwg != nullptr, "mole_gate_wgrad: null output");
    hipStream_t st = (hipStream_t)stream;
    ScopedTiming timing(MOLE_K_GATE_WGRAD, st);
    if (S == 0) {
        // no tokens: the reduction over zero partials writes the zeros (a kernel, not a memset, so that a
        // caller may capture the call in a graph)
        MOLE_REQUIRE(aligned16(dwg), "mole_gate_wgrad: misaligned output");
        hipLaunchKernelGGL(gate_wgrad_reduce_kernel, dim3(ceil_div(E * M, 64)), dim3(256), 0, st, (const float *)dwg, 0, E * M, dwg);
        MOLE_LAUNCH_CHECK();
        return 0;
    }
    MOLE_REQUIRE(dlogits && x && workspace && aligned16(x) && aligned16(dwg) && aligned16(workspace), "mole_gate_wgrad: null or misaligned pointer");
    if (workspace_bytes < mole_gate_wgrad_workspace_bytes(S, E, M)) {
        set_error("mole_gate_wgrad: workspace of %zu bytes, need %zu", workspace_bytes, mole_gate_wgrad_workspace_bytes(S, E, M));
        return MOLE_E_WORKSPACE;
    }
    float *part = (float *)workspace;
    if (gate_wgrad_mfma_ok(dtype, S, E, M)) {
        const int chunk = gate_wgrad_mfma_chunk(S, E, M), nchunks = ceil_div(S, chunk);
        const int eg = E <= 16 ? 1 : (E <= 32 ? 2 : 4);
        const int nz = ceil_div(E, 16 * eg), nunits = nchunks * ceil_div(M, 256);
        const dim3 grid((unsigned)(ceil_div(nunits, 8) * 8 * nz));
#define MOLE_GM(EG, V) hipLaunchKernelGGL((gate_wgrad_mfma_kernel<EG, V>), grid, dim3(256), 0, st, dlogits, (const bf16_t *)x, S, E, M, chunk, nchunks, nz, part)
        if (E % 4 == 0 && aligned16(dlogits)) {
            if (eg == 1) MOLE_GM(1, true); else if (eg == 2) MOLE_GM(2, true); else MOLE_GM(4, true);
        } else {
            if (eg == 1) MOLE_GM(1, false); else if (eg == 2) MOLE_GM(2, false); else MOLE_GM(4, false);
        }
#undef MOLE_GM
        MOLE_LAUNCH_CHECK();
        hipLaunchKernelGGL(gate_wgrad_reduce_kernel, dim3(ceil_div(E * M, 64)), dim3(256), 0, st, part, nchunks, E * M, dwg);
        MOLE_LAUNCH_CHECK();
        return 0;
    }
    const int nb = ceil_div(S, GW_TOKENS);
    const dim3 grid(nb, ceil_div(M, 512));
#define MOLE_GW(T, EB) hipLaunchKernelGGL((gate_wgrad_partial_kernel<T, EB>), grid, dim3(256), 0, st, dlogits, (const T *)x, S, E, M, part)
    if (dtype == MOLE_BF16) {
        if (E <= 8) MOLE_GW(bf16_t, 8); else if (E <= 16) MOLE_GW(bf16_t, 16); else MOLE_GW(bf16_t, 32);
    } else {
        if (E <= 8) MOLE_GW(float, 8); else if (E <= 16) MOLE_GW(float, 16); else MOLE_GW(float, 32);
    }
#undef MOLE_GW
    MOLE_LAUNCH_CHECK();
    hipLaunchKernelGGL(gate_wgrad_reduce_kernel, dim3(ceil_div(E * M, 64)), dim3(256), 0, st, part, nb, E * M, dwg);
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" int mole_combine_fwd(const void *o, int dtype, const int32_t *row, const float *gates, int S, int M,
                                int k, void *y, mole_stream_t stream) {
    if (int rc = check_perm("mole_combine_fwd", dtype, S, M, k)) return rc;
    if (S == 0) return 0;
    MOLE_REQUIRE(o && row && gates && y && aligned16(o) && aligned16(y), "mole_combine_fwd: null or misaligned pointer");
    if (dtype == MOLE_BF16)
        PM_LAUNCH_KT(MOLE_K_COMBINE_FWD, combine_fwd_kernel, bf16_t, 4, (const bf16_t *)o, row, gates, S, M, k, (bf16_t *)y);
    else
        PM_LAUNCH_KT(MOLE_K_COMBINE_FWD, combine_fwd_kernel, float, 4, (const float *)o, row, gates, S, M, k, (float *)y);
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" int mole_combine_bwd(const void *dy, const void *o, int dtype, const int32_t *row, const float *gates,
                                int S, int M, int k, void *d_o, float *dgates, mole_stream_t stream) {
    if (int rc = check_perm("mole_combine_bwd", dtype, S, M, k)) return rc;
    if (S == 0) return 0;
    MOLE_REQUIRE(dy && o && row && gates && d_o && dgates && aligned16(dy) && aligned16(o) && aligned16(d_o),
                 "mole_combine_bwd: null or misaligned pointer");
    const dim3 grid(ceil_div(S, PM_THREADS / WAVE));
    if (dtype == MOLE_BF16)
        PM_LAUNCH_K(MOLE_K_COMBINE_BWD, combine_bwd_kernel, bf16_t, (const bf16_t *)dy, (const bf16_t *)o, row, gates, S, M, k, (bf16_t *)d_o, dgates);
    else
        PM_LAUNCH_K(MOLE_K_COMBINE_BWD, combine_bwd_kernel, float, (const float *)dy, (const float *)o, row, gates, S, M, k, (float *)d_o, dgates);
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" int mole_combine_bwd_gate(const void *dy, const void *o, int dtype, const int32_t *row, const float *gates,
                                     int S, int M, int k, void *d_o, const float *scores, const int32_t *idx, int E,
                                     int normalize_gate, int through_softmax, const int32_t *counts0,
                                     const float *d_l_aux, float *dlogits, mole_stream_t stream) {
    if (int rc = check_perm("mole_combine_bwd_gate", dtype, S, M, k)) return rc;
    MOLE_REQUIRE(E >= 1 && E <= 256 && k <= E, "mole_combine_bwd_gate: E=%d must be 1..256 and at least k=%d (larger gates: mole_combine_bwd + mole_gate_bwd)", E, k);
    if (S == 0) return 0;
    MOLE_REQUIRE(dy && o && row && gates && d_o && scores && idx && dlogits && aligned16(dy) && aligned16(o) && aligned16(d_o),
                 "mole_combine_bwd_gate: null or misaligned pointer");
    MOLE_REQUIRE((counts0 == nullptr) == (d_l_aux == nullptr), "mole_combine_bwd_gate: counts0 and d_l_aux go together");
    const GateBwdArgs ga{scores, idx, E, normalize_gate, through_softmax, counts0, d_l_aux, dlogits};
    const dim3 grid(ceil_div(S, PM_THREADS / WAVE)), blk(PM_THREADS);
    hipStream_t st = (hipStream_t)stream;
    const int vpl = E <= 64 ? 1 : (E <= 128 ? 2 : 4);
#define MOLE_CBG(T, KK)                                                                                              \
    do {                                                                                                             \
        if (vpl == 1) timed_launch(MOLE_K_COMBINE_BWD, combine_bwd_gate_kernel<T, KK, 1>, grid, blk, 0, st, (const T *)dy, (const T *)o, row, gates, S, M, k, (T *)d_o, ga); \
        else if (vpl == 2) timed_launch(MOLE_K_COMBINE_BWD, combine_bwd_gate_kernel<T, KK, 2>, grid, blk, 0, st, (const T *)dy, (const T *)o, row, gates, S, M, k, (T *)d_o, ga); \
        else timed_launch(MOLE_K_COMBINE_BWD, combine_bwd_gate_kernel<T, KK, 4>, grid, blk, 0, st, (const T *)dy, (const T *)o, row, gates, S, M, k, (T *)d_o, ga); \
    } while (0)
#define MOLE_CBG_K(T)                                                                                                \
    do {                                                                                                             \
        if (k <= 1) MOLE_CBG(T, 1); else if (k <= 2) MOLE_CBG(T, 2); else if (k <= 4) MOLE_CBG(T, 4);                \
        else if (k <= 8) MOLE_CBG(T, 8); else MOLE_CBG(T, 16);                                                       \
    } while (0)
    if (dtype == MOLE_BF16) MOLE_CBG_K(bf16_t); else MOLE_CBG_K(float);
#undef MOLE_CBG_K
#undef MOLE_CBG
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" int mole_zero_pad_rows(void *buf, int dtype, const int32_t *kept_rows, const int32_t *offsets, int E,
                                  int M, mole_stream_t stream) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "mole_zero_pad_rows: bad dtype %d", dtype);
    MOLE_REQUIRE(E >= 1 && E <= MOLE_MAX_EXPERTS && M > 0 && M % (dtype == MOLE_BF16 ? 8 : 4) == 0,
                 "mole_zero_pad_rows: bad sizes E=%d M=%d", E, M);
    MOLE_REQUIRE(buf && kept_rows && offsets && aligned16(buf), "mole_zero_pad_rows: null or misaligned pointer");
    const dim3 grid(64, E);
    if (dtype == MOLE_BF16)
        hipLaunchKernelGGL(zero_pad_rows_kernel<bf16_t>, grid, dim3(PM_THREADS), 0, (hipStream_t)stream,
                           (bf16_t *)buf, kept_rows, offsets, M);
    else
        hipLaunchKernelGGL(zero_pad_rows_kernel<float>, grid, dim3(PM_THREADS), 0, (hipStream_t)stream,
                           (float *)buf, kept_rows, offsets, M);
    MOLE_LAUNCH_CHECK();
    return 0;
}
