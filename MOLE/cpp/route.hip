// Routing: top-k with lowest-index ties, gate values, per-expert counts, k-major locations,
// capacity and the dispatch permutation.  Deterministic: no atomics, every sum has a fixed order.
//
// Replaces tutel's extract_critical (called at MOLE/moe/layer.py:445-446) and the softmax half of
// MOLETopk.forward (MOLE/utils/Ugate.py:13).
//
// Four launches, all on the caller's stream:
//   route_topk      64 tokens per block (16 per wave).  A group of G lanes (G = pow2 >= E, at most 64) owns one
//                   token and holds VPL = ceil(E/G) scores per lane; k rounds of a shuffle arg-max
//                   with the (score desc, index asc) order.  Then, per choice j, the rank of each
//                   token among the block's earlier tokens with the same expert: wave ballot +
//                   popcount over the block's 64 tokens.
//   route_scan      one wave per (choice, expert): exclusive prefix over the blocks' histograms.
//   route_finish    one block: per-expert totals, capacity, kept rows, row offsets, l_aux.
//   route_finalize  loc = base(choice, expert) + block prefix + in-block rank; row = offset + loc.
#include "common.h"

#include <limits.h>
#include <math.h>

#include <mutex>
#include <stdlib.h>

namespace mole {

constexpr int RT_THREADS = 256;
constexpr int RT_TOKENS = 64;   // tokens per block: 16 per wave in the top-k phase; a choice is ranked by one wave over all 64
constexpr int RT_WTOK = RT_TOKENS / 4;
constexpr float FP32_EPS = 1.1920928955078125e-07f;

// A load that is always issued (the caller clamps the address to something valid) and gives +0 where the value
// must not count.  Written as "ok ? p[i] : 0" the load sits under a branch, and the compiler then waits for every
// load in flight at each such branch: a batch of loads meant to overlap runs one after the other.
__device__ __forceinline__ float load_or_zero(const float *p, bool ok) {
    return __uint_as_float(__float_as_uint(*p) & (ok ? 0xffffffffu : 0u));
}
__device__ __forceinline__ int load_or_zero(const int *p, bool ok) { return *p & (ok ? -1 : 0); }

// torch.topk's order of scores as an unsigned key: NaN ranks above everything and NaNs are equal among
// themselves, then +inf .. -inf with -0 == +0.  Every key of a real score is above 0, which stands for "not
// available" (outside the gate, or already chosen).  Equal keys are ranked by expert index, lowest first.
__device__ __forceinline__ uint32_t topk_key(float v) {
    uint32_t u = __float_as_uint(v);
    if (v != v) return 0xffffffffu;
    if (u == 0x80000000u) u = 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float topk_unkey(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

// max / min over aligned groups of 2^logG lanes, result in every lane of the group.  Within a row of 16 lanes the
// exchange is a DPP lane pattern (no LDS, no index registers): neighbours, pairs, then the mirrored half row and
// the mirrored row, each of which pairs a lane with one from the other already-reduced half.  32-lane groups add
// one crossbar swizzle, the whole wave reads the four row results into scalars.
template <int CTRL> __device__ __forceinline__ int dpp_lane(int x) {
    return __builtin_amdgcn_update_dpp(x, x, CTRL, 0xf, 0xf, false);
}
template <typename T, typename Op> __device__ __forceinline__ T group_reduce(T x, int logG, Op op) {
    static_assert(sizeof(T) == 4, "32-bit lanes");
    auto bits = [](T v) { return __builtin_bit_cast(int, v); };
    auto val = [](int v) { return __builtin_bit_cast(T, v); };
    if (logG >= 1) x = op(x, val(dpp_lane<0xb1>(bits(x))));      // quad_perm [1,0,3,2]
    if (logG >= 2) x = op(x, val(dpp_lane<0x4e>(bits(x))));      // quad_perm [2,3,0,1]
    if (logG >= 3) x = op(x, val(dpp_lane<0x141>(bits(x))));     // row_half_mirror
    if (logG >= 4) x = op(x, val(dpp_lane<0x140>(bits(x))));     // row_mirror
    if (logG == 5) x = op(x, val(__builtin_amdgcn_ds_swizzle(bits(x), 0x401f)));   // lane ^ 16 within 32 lanes
    if (logG >= 6) {
        const int xi = bits(x);
        x = op(op(val(__builtin_amdgcn_readlane(xi, 0)), val(__builtin_amdgcn_readlane(xi, 16))),
               op(val(__builtin_amdgcn_readlane(xi, 32)), val(__builtin_amdgcn_readlane(xi, 48))));
    }
    return x;
}

// What a block does once the top-k of its BT tokens (BT <= 64) lies in LDS - s_idx / s_graw [k][BT]: expert and raw
// gate value of every choice, s_col [4][E]: the four waves' column sums of the block's scores: the block's column sums
// out, gate values and indices out, then each choice's in-block ranks and per-expert histogram.  Four waves.
__device__ __forceinline__ void topk_block_tail(int BT, int S, int E, int k, int normalize, const int *s_idx,
                                                const float *s_graw, int *s_hist, const float *s_col,
                                                int32_t *__restrict__ idx, int32_t *__restrict__ lrank,
                                                float *__restrict__ gates, int32_t *__restrict__ hist,
                                                float *__restrict__ colsum, int nb) {
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int b = blockIdx.x, tok0 = b * BT;
    __syncthreads();
    for (int e = tid; e < E; e += RT_THREADS)
        colsum[(size_t)b * E + e] = ((s_col[e] + s_col[E + e]) + s_col[2 * E + e]) + s_col[3 * E + e];

    // ---- gate values and indices out (threads 0..BT-1 = the block's tokens) -------------
    const int token = tok0 + tid;
    const bool tv = tid < BT && token < S;
    if (tv) {
        float denom = 0.f;
        for (int j = 0; j < k; ++j) denom += s_graw[j * BT + tid];  // left to right, fp32
        const float den = denom < FP32_EPS ? FP32_EPS : denom;
        for (int j = 0; j < k; ++j) {
            float gv = s_graw[j * BT + tid];
            if (k > 1 && normalize) gv = gv / den;
            gates[(size_t)j * S + token] = gv;
            idx[(size_t)j * S + token] = s_idx[j * BT + tid];
        }
    }

    // ---- in-block ranks per choice (lane = token; wave w takes choices w, w + 4, ...) ------
    // Each wave works on a histogram of its own, so the choices proceed side by side without block barriers
    // (the loop over distinct experts is a serial chain of ballots: with one wave doing all k choices it was the
    // longest part of the kernel at top-8).
    const uint64_t lt_mask = (1ull << lane) - 1ull;
    int *my_hist = s_hist + w * E;
    const int ctoken = tok0 + lane;
    const bool cv = lane < BT && ctoken < S;
    for (int j = w; j < k; j += RT_THREADS / WAVE) {
        for (int e = lane; e < E; e += WAVE) my_hist[e] = 0;
        const int e = cv ? s_idx[j * BT + lane] : -1;
        int rank = 0;
        uint64_t remaining = __ballot(cv);
        while (remaining) {
            const int leader = __ffsll((unsigned long long)remaining) - 1;
            const int e0 = __shfl(e, leader, WAVE);
            const uint64_t m = __ballot(cv && e == e0);
            if (cv && e == e0) rank = __popcll(m & lt_mask);
            if (lane == leader) my_hist[e0] = __popcll(m);
            remaining &= ~m;
        }
        if (cv) lrank[(size_t)j * S + ctoken] = rank;
        // (the histogram is written and read by this wave only: program order is enough)
        for (int e2 = lane; e2 < E; e2 += WAVE) hist[((size_t)j * E + e2) * nb + b] = my_hist[e2];
    }
}

template <int VPL>
__global__ __launch_bounds__(RT_THREADS) void route_topk_kernel(
    const float *__restrict__ scores, int S, int E, int k, int logG, int normalize,
    int32_t *__restrict__ idx, int32_t *__restrict__ lrank, float *__restrict__ gates,
    int32_t *__restrict__ hist /* [k][E][nb] */, float *__restrict__ colsum /* [nb][E] */, int nb) {
    extern __shared__ char smem[];
    int *s_idx = (int *)smem;                          // [k][64]
    float *s_graw = (float *)(s_idx + k * RT_TOKENS);  // [k][64]
    int *s_hist = (int *)(s_graw + k * RT_TOKENS);     // [4][E]: one histogram per wave
    float *s_col = (float *)(s_hist + 4 * E);          // [4][E]

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int b = blockIdx.x, tok0 = b * RT_TOKENS;
    const int G = 1 << logG;
    const int tpw = 64 >> logG;  // tokens a wave handles per pass
    const int g = lane & (G - 1), tg = lane >> logG;

    // ---- phase A: top-k of every token (wave w owns tokens 16w .. 16w+15 of the block) ----------
    float colacc[VPL];
#pragma unroll
    for (int r = 0; r < VPL; ++r) colacc[r] = 0.f;

    // the scores of the wave's next token(s) are fetched while the current ones go through their k rounds
    float nxt[VPL];
#pragma unroll
    for (int r = 0; r < VPL; ++r) nxt[r] = 0.f;
    auto fetch = [&](int it) __attribute__((always_inline)) {
        const int tok = min(tok0 + w * RT_WTOK + it * tpw + tg, S - 1);
#pragma unroll
        for (int r = 0; r < VPL; ++r) nxt[r] = scores[(size_t)tok * E + min(g + (r << logG), E - 1)];
    };
    if (S > 0) fetch(0);
    for (int it = 0; it * tpw < RT_WTOK; ++it) {
        const int tw = it * tpw + tg;                  // token within the wave's 16
        const int tl = w * RT_WTOK + tw;
        const int token = tok0 + tl;
        const bool tv = tw < RT_WTOK && token < S;
        uint32_t key[VPL];
#pragma unroll
        for (int r = 0; r < VPL; ++r) {
            const bool ok = tv && g + (r << logG) < E;
            const float sv = __uint_as_float(__float_as_uint(nxt[r]) & (ok ? 0xffffffffu : 0u));
            colacc[r] += sv;
            key[r] = ok ? topk_key(sv) : 0u;
        }
        if (S > 0 && (it + 1) * tpw < RT_WTOK) fetch(it + 1);
        for (int j = 0; j < k; ++j) {
            // the best score of the token, then the lowest expert index among those that hold it
            uint32_t best = key[0];
#pragma unroll
            for (int r = 1; r < VPL; ++r) best = max(best, key[r]);
            const uint32_t top = group_reduce(best, logG, [](uint32_t a, uint32_t c) { return max(a, c); });
            int cand = INT_MAX;
#pragma unroll
            for (int r = VPL - 1; r >= 0; --r)
                if (key[r] == top) cand = g + (r << logG);             // ends on the lane's lowest such expert
            if (top == 0u) cand = INT_MAX;                             // nothing available (a token past the end)
            const int bi = group_reduce(cand, logG, [](int a, int c) { return min(a, c); });
            const bool mine = bi != INT_MAX && (bi & (G - 1)) == g;
#pragma unroll
            for (int r = 0; r < VPL; ++r)
                if (mine && (bi >> logG) == r) key[r] = 0u;
            if (g == 0 && tv) {
                s_idx[j * RT_TOKENS + tl] = bi;
                s_graw[j * RT_TOKENS + tl] = topk_unkey(top);
            }
        }
    }
    // column sums of the scores (for l_aux): fold the token groups of a wave, then the 4 waves
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        float c = colacc[r];
        for (int m = G; m < WAVE; m <<= 1) c += __shfl_xor(c, m, WAVE);
        const int e = g + (r << logG);
        if (tg == 0 && e < E) s_col[w * E + e] = c;
    }
    topk_block_tail(RT_TOKENS, S, E, k, normalize, s_idx, s_graw, s_hist, s_col, idx, lrank, gates, hist, colsum, nb);
}

// one wave per (choice, expert) pair: exclusive prefix over blocks, total into counts
__device__ __forceinline__ void scan_pair(int32_t *__restrict__ hist, int nb, int pair, int32_t *__restrict__ counts) {
    const int lane = threadIdx.x & 63;
    int carry = 0;
    // four chunks of 64 blocks at a time: their loads are in flight together
    for (int c0 = 0; c0 < nb; c0 += 4 * WAVE) {
        int v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int bi = c0 + u * WAVE + lane;
            v[u] = load_or_zero(hist + (size_t)pair * nb + min(bi, nb - 1), bi < nb);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int bi = c0 + u * WAVE + lane;
            int x = v[u];
            for (int d = 1; d < WAVE; d <<= 1) {
                const int y = __shfl_up(x, d, WAVE);
                if (lane >= d) x += y;
            }
            if (bi < nb) hist[(size_t)pair * nb + bi] = carry + x - v[u];
            carry += __shfl(x, WAVE - 1, WAVE);
        }
    }
    if (lane == 0) counts[pair] = carry;
}
// Blocks past the scan's own fold the per-block column sums of the scores (for l_aux) into COLSUM_SLICES rows:
// slice s adds blocks s, s + COLSUM_SLICES, ... in that order, so the single block that finishes the routing
// reads COLSUM_SLICES rows instead of one per 64 tokens (at 32768 tokens and 256 experts that loop was 40 us).
constexpr int COLSUM_SLICES = 16;
__global__ __launch_bounds__(256) void route_scan_kernel(int32_t *__restrict__ hist, int nb, int npairs,
                                                         int32_t *__restrict__ counts, int scan_blocks,
                                                         const float *__restrict__ colsum, int E,
                                                         float *__restrict__ colpart) {
    if ((int)blockIdx.x < scan_blocks) {
        const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);
        if (pair < npairs) scan_pair(hist, nb, pair, counts);
        return;
    }
    const int cb = blockIdx.x - scan_blocks;
    const int slice = cb % COLSUM_SLICES, e = (cb / COLSUM_SLICES) * 256 + threadIdx.x;
    if (e >= E) return;
    float me = 0.f;
    for (int b0 = slice; b0 < nb; b0 += 8 * COLSUM_SLICES) {        // 8 loads in flight, added in block order
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int b = b0 + u * COLSUM_SLICES;
            t[u] = load_or_zero(colsum + (size_t)min(b, nb - 1) * E + e, b < nb);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (b0 + u * COLSUM_SLICES < nb) me += t[u];
    }
    colpart[slice * E + e] = me;
}

constexpr int FIN_THREADS = 1024;

// scan_hist != NULL: the block first does the work of route_scan_kernel itself (small problems: one launch
// less), its 16 waves taking the pairs in turn.
__global__ __launch_bounds__(FIN_THREADS) void route_finish_kernel(
    int32_t *__restrict__ counts, const float *__restrict__ colsum, int nb, int S, int E, int k,
    int cf_sign, int cap_bound, int alignment, int layout, int32_t *__restrict__ basej,
    int32_t *__restrict__ kept_rows, int32_t *__restrict__ offsets, int32_t *__restrict__ capacity,
    float *__restrict__ l_aux, int32_t *__restrict__ scan_hist) {
    __shared__ int s_n[MOLE_MAX_EXPERTS];
    __shared__ int s_red[FIN_THREADS];
    __shared__ float s_fred[FIN_THREADS];
    const int tid = threadIdx.x;
    if (scan_hist != nullptr) {
        for (int pair = tid >> 6; pair < k * E; pair += FIN_THREADS / 64) scan_pair(scan_hist, nb, pair, counts);
        __threadfence_block();
        __syncthreads();
    }
    // only the first min(E, FIN_THREADS) threads hold data: the block-wide reductions and the scan below run over
    // the next power of two, not over all 1024 threads (fewer barrier rounds for small gates)
    int P = 1;
    while (P < E && P < FIN_THREADS) P <<= 1;
    int lmax = 0;
    for (int e = tid; e < E; e += FIN_THREADS) {
        int tot = 0;
        for (int j = 0; j < k; ++j) {
            basej[j * E + e] = tot;
            tot += counts[j * E + e];
        }
        s_n[e] = tot;
        lmax = max(lmax, tot);
    }
    s_red[tid] = lmax;
    __syncthreads();
    for (int d = P / 2; d >= 1; d >>= 1) {
        if (tid < d) s_red[tid] = max(s_red[tid], s_red[tid + d]);
        __syncthreads();
    }
    int cap = cf_sign > 0 ? cap_bound : s_red[0];
    if (cf_sign < 0) cap = min(cap, cap_bound);
    const int rem = cap % alignment;
    if (rem > 0) cap += alignment - rem;
    __syncthreads();

    // kept rows, then their exclusive prefix (chunk per thread + Hillis-Steele over the chunks)
    const int chunk = (E + FIN_THREADS - 1) / FIN_THREADS;
    const int lo = min(tid * chunk, E), hi = min(lo + chunk, E);
    int csum = 0;
    for (int e = lo; e < hi; ++e) {
        const int n = min(s_n[e], cap);
        s_n[e] = n;
        kept_rows[e] = n;
        csum += n;
    }
    s_red[tid] = csum;
    __syncthreads();
    for (int d = 1; d < P; d <<= 1) {
        const int y = tid >= d ? s_red[tid - d] : 0;
        __syncthreads();
        s_red[tid] += y;
        __syncthreads();
    }
    if (layout == MOLE_LAYOUT_RAGGED) {
        int run = s_red[tid] - csum;
        for (int e = lo; e < hi; ++e) {
            offsets[e] = run;
            run += s_n[e];
        }
        if (tid == P - 1) offsets[E] = s_red[tid];
    } else {
        for (int e = lo; e < hi; ++e) offsets[e] = e * cap;
        if (tid == 0) offsets[E] = E * cap;
    }
    if (tid == 0) capacity[0] = cap;

    if (l_aux != nullptr) {
        // me[e] = sum over blocks of the partial column sums, in a fixed order: thread (g, e) adds
        // blocks g, g+groups, ...; thread e then adds the groups in order
        __syncthreads();
        const int groups = FIN_THREADS / E > 0 ? FIN_THREADS / E : 1;
        if (tid < groups * E && E <= FIN_THREADS) {
            const int e = tid % E, gq = tid / E;
            float me = 0.f;
            for (int b0 = gq; b0 < nb; b0 += 8 * groups) {       // 8 loads in flight, added in block order
                float t[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int b = b0 + u * groups;
                    t[u] = load_or_zero(colsum + (size_t)min(b, nb - 1) * E + e, b < nb);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (b0 + u * groups < nb) me += t[u];
            }
            s_fred[tid] = me;
        }
        __syncthreads();
        float acc = 0.f;
        if (tid < E) {
            float me = 0.f;
            for (int gq = 0; gq < groups; ++gq) me += s_fred[gq * E + tid];
            acc = me * (float)counts[tid];
        }
        __syncthreads();
        s_fred[tid] = acc;
        __syncthreads();
        for (int d = P / 2; d >= 1; d >>= 1) {
            if (tid < d) s_fred[tid] += s_fred[tid + d];
            __syncthreads();
        }
        if (tid == 0) l_aux[0] = S > 0 ? s_fred[0] * ((float)E / ((float)S * (float)S)) : 0.f;
    }
}

__global__ __launch_bounds__(256) void route_finalize_kernel(
    const int32_t *__restrict__ idx, const int32_t *__restrict__ hist, const int32_t *__restrict__ basej,
    const int32_t *__restrict__ offsets, const int32_t *__restrict__ capacity, int S, int E, int k, int nb,
    int bt /* tokens per histogram block */, int32_t *__restrict__ loc /* in: in-block rank, out: location */,
    int32_t *__restrict__ row) {
    const size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= (size_t)k * S) return;
    const int j = (int)(p / S), i = (int)(p % S);
    const int e = idx[p];
    const int b = i / bt;
    const int l = basej[j * E + e] + hist[((size_t)j * E + e) * nb + b] + loc[p];
    loc[p] = l;
    row[p] = l < capacity[0] ? offsets[e] + l : -1;
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace mole

using namespace mole;

extern "C" size_t mole_route_workspace_bytes(int S, int E, int k) {
    if (S < 0 || E <= 0 || k <= 0) return 0;
    const size_t nb = (size_t)ceil_div(S > 0 ? S : 1, RT_TOKENS);
    return align256(nb * k * E * sizeof(int32_t)) + align256((size_t)k * E * sizeof(int32_t)) +
           align256(nb * E * sizeof(float)) + align256((size_t)COLSUM_SLICES * E * sizeof(float));
}

// Lanes per token (as a power of two) of the kernels that give a group of lanes a token's E values, each lane holding
// E / lanes of them: 16 lanes at most, more only where a lane would otherwise hold more than 16 values.  A group's
// reductions act on all the wave's groups at once, so in the top-k, whose rounds are chains of reductions, small groups
// with many values per lane cost fewer instructions per token than the whole wave on one token (top-8 of 256 scores for 32768 tokens: 106 us with 64 lanes per token,
// 83 with 32, 72 with 16; top-2 of 64 for 8192: 33.6 / 29.5 / 25.8 us).
static int lane_group_log2(int E) {
    int logG = 0;
    while ((1 << logG) < E && logG < 4) ++logG;
    while (ceil_div(E, 1 << logG) > 16 && logG < 6) ++logG;
    return logG;
}

// The stages of the routing behind the per-block top-k: scan of the histograms over blocks, counts / capacity /
// offsets / l_aux, then locations and destination rows.  bt: tokens per histogram block.
static int route_after_topk(int32_t *hist, int32_t *basej, float *colsum, float *colpart, int nb, int bt, int S, int E, int k,
                            double capacity_factor, int alignment, int layout, const int32_t *idx, int32_t *loc,
                            int32_t *row, int32_t *counts, int32_t *kept_rows, int32_t *offsets, int32_t *capacity,
                            float *l_aux, hipStream_t st) {
    const int npairs = k * E;
    const bool scan_in_finish = (long long)npairs * nb <= 8192;    // small enough for one block: saves a launch
    if (!scan_in_finish) {
        const int scan_blocks = ceil_div(npairs, 4);
        hipLaunchKernelGGL(route_scan_kernel, dim3(scan_blocks + COLSUM_SLICES * ceil_div(E, 256)), dim3(256), 0, st, hist,
                           nb, npairs, counts, scan_blocks, colsum, E, colpart);
        MOLE_LAUNCH_CHECK();
    }

    const int spe = (S + E - 1) / E;
    const int cf_sign = capacity_factor > 0. ? 1 : (capacity_factor < 0. ? -1 : 0);
    // int(cf * spe) of the Python reference: the product is taken in double precision
    const double prod = (capacity_factor < 0. ? -capacity_factor : capacity_factor) * (double)spe;
    const int cap_bound = k * (int)prod;
    // (when the scan kernel ran, it also folded the column sums: the finish then adds its COLSUM_SLICES rows)
    hipLaunchKernelGGL(route_finish_kernel, dim3(1), dim3(FIN_THREADS), 0, st, counts,
                       scan_in_finish ? colsum : colpart, scan_in_finish ? nb : min(nb, COLSUM_SLICES), S, E, k, cf_sign,
                       cap_bound, alignment, layout, basej, kept_rows, offsets, capacity, l_aux,
                       scan_in_finish ? hist : (int32_t *)nullptr);
    MOLE_LAUNCH_CHECK();

    if (S > 0) {
        const size_t n = (size_t)k * S;
        hipLaunchKernelGGL(route_finalize_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, idx, hist,
                           basej, offsets, capacity, S, E, k, nb, bt, loc, row);
        MOLE_LAUNCH_CHECK();
    }
    return 0;
}

template <int VPL>
static void launch_topk(const float *scores, int S, int E, int k, int logG, int normalize, int32_t *idx,
                        int32_t *loc, float *gates, int32_t *hist, float *colsum, int nb, hipStream_t st) {
    const size_t lds = (size_t)k * RT_TOKENS * 8 + (size_t)E * 4 * 4 + (size_t)E * 4 * 4;
    hipLaunchKernelGGL(route_topk_kernel<VPL>, dim3(nb), dim3(RT_THREADS), lds, st, scores, S, E, k, logG,
                       normalize, idx, loc, gates, hist, colsum, nb);
}

extern "C" int mole_route(const float *scores, int S, int E, int k, double capacity_factor, int normalize_gate,
                          int alignment, int layout, int32_t *idx, int32_t *loc, float *gates, int32_t *row,
                          int32_t *counts, int32_t *kept_rows, int32_t *offsets, int32_t *capacity,
                          float *l_aux, void *workspace, size_t workspace_bytes, mole_stream_t stream) {
    MOLE_REQUIRE(S >= 0 && E >= 1 && E <= MOLE_MAX_EXPERTS, "mole_route: need S >= 0 and 1 <= E <= %d (S=%d E=%d)",
                 MOLE_MAX_EXPERTS, S, E);
    MOLE_REQUIRE(k >= 1 && k <= MOLE_MAX_TOPK && k <= E, "mole_route: need 1 <= k <= min(E, %d) (k=%d E=%d)",
                 MOLE_MAX_TOPK, k, E);
    MOLE_REQUIRE(alignment >= 1, "mole_route: alignment must be >= 1");
    MOLE_REQUIRE(layout == MOLE_LAYOUT_PADDED || layout == MOLE_LAYOUT_RAGGED, "mole_route: bad layout %d", layout);
    MOLE_REQUIRE(counts && kept_rows && offsets && capacity && workspace, "mole_route: null output pointer");
    MOLE_REQUIRE(S == 0 || (scores && idx && loc && gates && row), "mole_route: null token buffer");
    MOLE_REQUIRE((long long)S * k < INT_MAX && (long long)S * E < (1ll << 40), "mole_route: S*k too large");
    if (workspace_bytes < mole_route_workspace_bytes(S, E, k)) {
        set_error("mole_route: workspace of %zu bytes, need %zu", workspace_bytes, mole_route_workspace_bytes(S, E, k));
        return MOLE_E_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    ScopedTiming timing(MOLE_K_ROUTE, st);
    const int nb = ceil_div(S > 0 ? S : 1, RT_TOKENS);
    char *ws = (char *)workspace;
    int32_t *hist = (int32_t *)ws;
    ws += align256((size_t)nb * k * E * sizeof(int32_t));
    int32_t *basej = (int32_t *)ws;
    ws += align256((size_t)k * E * sizeof(int32_t));
    float *colsum = (float *)ws;
    ws += align256((size_t)nb * E * sizeof(float));
    float *colpart = (float *)ws;

    const int logG = lane_group_log2(E);
    const int vpl = ceil_div(E, 1 << logG);
    if (vpl <= 1) launch_topk<1>(scores, S, E, k, logG, normalize_gate, idx, loc, gates, hist, colsum, nb, st);
    else if (vpl <= 2) launch_topk<2>(scores, S, E, k, logG, normalize_gate, idx, loc, gates, hist, colsum, nb, st);
    else if (vpl <= 4) launch_topk<4>(scores, S, E, k, logG, normalize_gate, idx, loc, gates, hist, colsum, nb, st);
    else if (vpl <= 8) launch_topk<8>(scores, S, E, k, logG, normalize_gate, idx, loc, gates, hist, colsum, nb, st);
    else launch_topk<16>(scores, S, E, k, logG, normalize_gate, idx, loc, gates, hist, colsum, nb, st);
    MOLE_LAUNCH_CHECK();

    return route_after_topk(hist, basej, colsum, colpart, nb, RT_TOKENS, S, E, k, capacity_factor, alignment, layout, idx, loc,
                            row, counts, kept_rows, offsets, capacity, l_aux, st);
}

// ---------------------------------------------------------------------------------------------
// mole_route without a workspace argument and without any allocation: the per-block histograms, the per-choice
// bases and the column sums of the scores live in a file-scope device array.  Each GPU the library runs on holds
// its own copy of the array until the process ends.  The array's name is only a host-side handle; the address
// the kernels get is looked up once per device with hipGetSymbolAddress and kept.
// ---------------------------------------------------------------------------------------------
#define MOLE_ROUTE_SCRATCH_BYTES (8u << 20)
static __device__ __align__(256) unsigned char scratch[MOLE_ROUTE_SCRATCH_BYTES];

namespace mole {
constexpr int MAX_SCRATCH_DEVICES = 64;
static void *g_scratch_ptr[MAX_SCRATCH_DEVICES];
static std::mutex g_scratch_mu;

// device address of `scratch` on the current device
static int route_scratch(void **out) {
    int dev = 0;
    MOLE_HIP(hipGetDevice(&dev));
    MOLE_REQUIRE(dev >= 0 && dev < MAX_SCRATCH_DEVICES, "mole_route_static: device %d out of range", dev);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        MOLE_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        MOLE_REQUIRE(p != nullptr, "mole_route_static: hipGetSymbolAddress returned no address");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
}  // namespace mole

extern "C" size_t mole_route_static_max_bytes(void) { return MOLE_ROUTE_SCRATCH_BYTES; }

extern "C" int mole_route_static(const float *scores, int S, int E, int k, double capacity_factor, int normalize_gate,
                                 int alignment, int layout, int32_t *idx, int32_t *loc, float *gates, int32_t *row,
                                 int32_t *counts, int32_t *kept_rows, int32_t *offsets, int32_t *capacity, float *l_aux,
                                 mole_stream_t stream) {
    const size_t need = mole_route_workspace_bytes(S, E, k);
    if (need == 0 || need > MOLE_ROUTE_SCRATCH_BYTES) {
        set_error("mole_route_static: S=%d E=%d k=%d needs %zu bytes of scratch, the static array holds %zu "
                  "(use mole_route with a workspace of your own)", S, E, k, need, (size_t)MOLE_ROUTE_SCRATCH_BYTES);
        return need == 0 ? MOLE_E_INVALID : MOLE_E_WORKSPACE;
    }
    void *ptr = nullptr;
    if (int rc = route_scratch(&ptr)) return rc;
    // every word of the scratch that a kernel of the route reads has been written by an earlier kernel of the
    // same call (the histograms by the top-k blocks, the bases and column sums by the scan / finish kernels), so
    // nothing needs clearing between calls; calls that overlap on one GPU would race on it
    return mole_route(scores, S, E, k, capacity_factor, normalize_gate, alignment, layout, idx, loc, gates, row, counts,
                      kept_rows, offsets, capacity, l_aux, ptr, MOLE_ROUTE_SCRATCH_BYTES, stream);
}

// ---------------------------------------------------------------------------------------------
// softmax over experts (MOLE/utils/Ugate.py:13) and the backward from dgates to dlogits
// ---------------------------------------------------------------------------------------------
namespace mole {

// One group of G lanes per token (same mapping as route_topk), VPL values per lane.
template <int VPL>
__global__ __launch_bounds__(256) void softmax_fwd_kernel(const float *__restrict__ logits,
                                                          const float *__restrict__ bias, int S, int E, int logG,
                                                          float *__restrict__ scores) {
    const int lane = threadIdx.x & 63;
    const int G = 1 << logG;
    const int g = lane & (G - 1), tg = lane >> logG;
    const int tpw = 64 >> logG;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int token = wave * tpw + tg;
    const bool tv = token < S;
    float v[VPL];
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = g + (r << logG);
        const bool ok = tv && e < E;
        // (an unconditional load from a clamped address; entries that do not exist become -inf)
        const float lg = load_or_zero(logits + (size_t)min(token, S - 1) * E + min(e, E - 1), ok);
        v[r] = lg + (ok ? (bias ? bias[e] : 0.f) : -INFINITY);
        mx = fmaxf(mx, v[r]);
    }
    mx = group_reduce(mx, logG, [](float a, float c) { return fmaxf(a, c); });
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = g + (r << logG);
        v[r] = (tv && e < E) ? expf(v[r] - mx) : 0.f;
        sum += v[r];
    }
    sum = group_reduce(sum, logG, [](float a, float c) { return a + c; });
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = g + (r << logG);
        if (tv && e < E) scores[(size_t)token * E + e] = v[r] / sum;
    }
}

// Softmax backward on its own (the gate used outside the fused layer node): dlogits = s * (ds - sum_e ds s).
template <int VPL>
__global__ __launch_bounds__(256) void softmax_bwd_kernel(const float *__restrict__ dscores,
                                                          const float *__restrict__ scores, int S, int E, int logG,
                                                          float *__restrict__ dlogits) {
    const int lane = threadIdx.x & 63;
    const int G = 1 << logG;
    const int g = lane & (G - 1), tg = lane >> logG;
    const int tpw = 64 >> logG;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int token = wave * tpw + tg;
    const bool tv = token < S;
    float s[VPL], ds[VPL];
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = g + (r << logG);
        const size_t at = (size_t)min(token, S - 1) * E + min(e, E - 1);
        s[r] = load_or_zero(scores + at, tv && e < E);
        ds[r] = load_or_zero(dscores + at, tv && e < E);
        dot += ds[r] * s[r];
    }
    dot = group_reduce(dot, logG, [](float a, float c) { return a + c; });
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = g + (r << logG);
        if (tv && e < E) dlogits[(size_t)token * E + e] = s[r] * (ds[r] - dot);
    }
}

// dlogits[i,e] = s[i,e] * (dscore[i,e] - sum_e' dscore[i,e'] s[i,e']), dscore scattered from dgates
// through gate_j = graw_j / max(sum graw, eps).  The token's group of lanes shares the k-sized part, then
// writes the row.  With counts0 and d_l_aux given, dscore also carries the load-balancing loss
// l_aux = E/S^2 sum_e (sum_i s[i,e]) counts0[e]: d l_aux / d s[i,e] = E/S^2 counts0[e], the same for every token
// (the counts are integers and carry no gradient).
template <int VPL>
__global__ __launch_bounds__(256) void gate_bwd_kernel(const float *__restrict__ dgates,
                                                       const float *__restrict__ scores,
                                                       const int32_t *__restrict__ idx, int S, int E, int k,
                                                       int logG, int normalize, int through_softmax,
                                                       const int32_t *__restrict__ counts0,
                                                       const float *__restrict__ d_l_aux,
                                                       float *__restrict__ dlogits) {
    const int lane = threadIdx.x & 63;
    const int G = 1 << logG;
    const int g = lane & (G - 1), tg = lane >> logG;
    const int tpw = 64 >> logG;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int token = wave * tpw + tg;
    const bool tv = token < S;
    float s[VPL], ds[VPL];
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = g + (r << logG);
        s[r] = load_or_zero(scores + (size_t)min(token, S - 1) * E + min(e, E - 1), tv && e < E);
        ds[r] = 0.f;
    }
    if (counts0 != nullptr) {       // uniform over the grid
        const float scale = d_l_aux[0] * ((float)E / ((float)S * (float)S));
#pragma unroll
        for (int r = 0; r < VPL; ++r) ds[r] = scale * (float)counts0[min(g + (r << logG), E - 1)];
    }
    // Lane j < k of the token's group fetches choice j (index, incoming gradient, raw gate value), the sums over
    // the k choices are lane reductions, and each choice is then handed round the group.  (With every lane walking
    // the k choices itself the token paid 2 k dependent memory latencies.)
    const bool has = tv && g < k;
    const int tokc = min(token, S - 1), jc = min(g, k - 1);
    const int my_e = idx[(size_t)jc * S + tokc];
    const float my_dg = load_or_zero(dgates + (size_t)jc * S + tokc, has);
    const float my_gr = load_or_zero(scores + (size_t)tokc * E + min(max(my_e, 0), E - 1), has);
    const float denom = group_reduce(my_gr, logG, [](float a, float c) { return a + c; });
    const float dotg = group_reduce(my_dg * my_gr, logG, [](float a, float c) { return a + c; });
    const bool norm = k > 1 && normalize;
    const bool clamped = denom < FP32_EPS;
    const float den = clamped ? FP32_EPS : denom;
    const float sub = (norm && !clamped) ? dotg / (den * den) : 0.f;
    const float my_dgraw = norm ? my_dg / den - sub : my_dg;
    const int group_base = lane & ~(G - 1);
    for (int j = 0; j < k; ++j) {
        int e;
        float dgraw;
        if (logG >= 6) {       // the group is the wave: lane j is a scalar read
            e = __builtin_amdgcn_readlane(my_e, j);
            dgraw = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_dgraw), j));
        } else {
            e = __shfl(my_e, group_base + j, WAVE);
            dgraw = __shfl(my_dgraw, group_base + j, WAVE);
        }
        if ((e & (G - 1)) == g) {
            const int rr = e >> logG;
#pragma unroll
            for (int r = 0; r < VPL; ++r)
                if (r == rr) ds[r] += dgraw;
        }
    }
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) dot += ds[r] * s[r];
    dot = group_reduce(dot, logG, [](float a, float c) { return a + c; });
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
        const int e = g + (r << logG);
        if (tv && e < E) dlogits[(size_t)token * E + e] = through_softmax ? s[r] * (ds[r] - dot) : ds[r];
    }
}


// ---- the gate for fp32 tokens and small gates (E <= 32): one wave per token ------------------------------
// Lane l holds 4 columns of the token per pass (M / 256 passes) and accumulates its share of all E logits in
// registers against the matching columns of Wg (16-64 KB in all: L1/L2 hits); the E sums are reduced over the
// wave with lane patterns, lane e keeps logit e, and the softmax runs over the wave.  fp32 FMAs throughout.
// (The two-kernel path spends 44 us on a 4096 x 512 x 8 product: one 128 x 128 tile of the GEMM kernel per 128
// tokens leaves most of the chip idle.)
template <int EB>
__global__ __launch_bounds__(256) void gate_fwd_f32_kernel(const float *__restrict__ x, const float *__restrict__ wg,
                                                           const float *__restrict__ bias, int S, int E, int M,
                                                           float *__restrict__ scores) {
    const int lane = threadIdx.x & 63;
    const int token = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (token >= S) return;                       // a whole wave
    float acc[EB];
#pragma unroll
    for (int e = 0; e < EB; ++e) acc[e] = 0.f;
    const float *xr = x + (size_t)token * M;
    for (int c = lane * 4; c < M; c += 256) {
        const float4 xv = *reinterpret_cast<const float4 *>(xr + c);
#pragma unroll
        for (int e = 0; e < EB; ++e) {            // rows past the gate repeat its last row and are not used
            const float4 wv = *reinterpret_cast<const float4 *>(wg + (size_t)min(e, E - 1) * M + c);
            acc[e] = fmaf(xv.w, wv.w, fmaf(xv.z, wv.z, fmaf(xv.y, wv.y, fmaf(xv.x, wv.x, acc[e]))));
        }
    }
    float mine = -INFINITY;
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        const float sum = group_reduce(acc[e], 6, [](float a, float c) { return a + c; });
        if (lane == e && e < E) mine = sum + (bias ? bias[e] : 0.f);
    }
    const float mx = group_reduce(mine, 6, [](float a, float c) { return fmaxf(a, c); });
    const float ex = lane < E ? expf(mine - mx) : 0.f;
    const float den = group_reduce(ex, 6, [](float a, float c) { return a + c; });
    if (lane < E) scores[(size_t)token * E + lane] = ex / den;
}

// ---- fused gate: scores = softmax(x . Wg^T + bias) for bf16 tokens ------------------------------------
// A block of four waves owns 16 tokens; wave w contracts the w-th quarter of the model dimension with
// v_mfma_f32_16x16x32_bf16 (16 tokens x 16 experts x 32 of k per instruction), operands straight from
// global memory in the instruction's layout - lane l supplies 8 consecutive k (k slice l / 16) of token or
// expert l % 16 - with the fp32 gate weights rounded to bf16 on the fly, as the separate GEMM did.  The
// four partial logit tiles meet in LDS, then 16 lanes per token do the softmax.  EG = groups of 16 experts.
typedef __bf16 gate_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gate_f32x4 __attribute__((ext_vector_type(4)));

// STAGE: the token rows of a round reach the fragments by way of LDS.  Straight from memory, a load instruction of
// the instruction's layout touches 16 rows with 64 bytes each; staged, it fetches 512-byte pieces of two rows (at
// KSTEPS 8), and the fragments are 16-byte LDS reads (rows 16 bytes longer than their data: the 16 rows of a read
// fall into distinct banks).  A wave stages and reads its own rows only.
// ROUTE: the block goes on to the first stage of the routing for its 16 TG tokens - top-k, gate values, in-block
// ranks and per-expert histograms, the block's column sums for l_aux - while a token's scores are still in the 16
// lanes that formed them (the layout route_topk_kernel works in: lane j of the group holds experts j, 16 + j, ...).
// The scores are written out as well (the backward needs them) but not read back: one kernel and 4 S E bytes less.
struct GateRoute {
    int k, normalize, nb;
    int32_t *idx, *lrank, *hist;
    float *gates, *colsum;
};
template <int EG, int KSTEPS, int TG, bool STAGE, bool ROUTE = false>   // TG groups of 16 tokens per block: Wg is read once for all of them
__global__ __launch_bounds__(256) void gate_fwd_kernel(const bf16_t *__restrict__ x, const float *__restrict__ wg,
                                                       const float *__restrict__ bias, int S, int E, int M,
                                                       float *__restrict__ scores, const GateRoute rt) {
    constexpr int RB = KSTEPS * 64, RS = RB + 16;               // staged row: bytes of data, bytes of stride
    constexpr int LPR = RB / 16, RPI = 64 / LPR;                // lanes per row, rows per load instruction
    constexpr int PART_BYTES = 4 * 16 * TG * (EG * 16 + 1) * 4;
    constexpr int STAGE_BYTES = STAGE ? 4 * 16 * TG * RS : 0;
    static_assert(!STAGE || STAGE_BYTES >= PART_BYTES, "the launch sizes the dynamic LDS for the staged rows");
    __shared__ __align__(16) char s_static[STAGE ? 16 : PART_BYTES];
    extern __shared__ __align__(16) char s_dyn[];               // STAGE: max(PART_BYTES, STAGE_BYTES), given at launch
    char *s_all = STAGE ? s_dyn : s_static;
    float (*part)[16 * TG][EG * 16 + 1] = reinterpret_cast<float (*)[16 * TG][EG * 16 + 1]>(s_all);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int tok0 = blockIdx.x * 16 * TG;
    const int kbase = wave * (M >> 2) + 8 * kq;
    const bf16_t *xp[TG];
#pragma unroll
    for (int tg = 0; tg < TG; ++tg) xp[tg] = x + (size_t)min(tok0 + 16 * tg + r16, S - 1) * M + kbase;
    gate_f32x4 acc[TG][EG];
#pragma unroll
    for (int tg = 0; tg < TG; ++tg)
#pragma unroll
        for (int g = 0; g < EG; ++g) acc[tg][g] = gate_f32x4{0.f, 0.f, 0.f, 0.f};
    const int nsteps = M >> 7;                    // 32 of k per step, a quarter of M per wave
    // All loads of a round of KSTEPS steps go out first, unconditionally (a step past the end repeats the last
    // one and is masked below): under a condition each load would be waited for before the next is issued.  For
    // small gates the weights of the round are fetched ahead as well.
    constexpr bool W_AHEAD = EG * KSTEPS <= 16;
    for (int s0 = 0; s0 < nsteps; s0 += KSTEPS) {
        uint4 a[TG][KSTEPS];
        float4 wa[W_AHEAD ? KSTEPS : 1][W_AHEAD ? EG : 1][2];
        if constexpr (STAGE) {
            // load j of the round: rows RPI j + lane / LPR of the block's 16 TG, 16 bytes at (lane % LPR) 16 of the
            // round's RB; columns past the wave's quarter (steps past the end) repeat its last 16 bytes
            const int cb = min(s0 * 32 + (lane % LPR) * 8, (M >> 2) - 8);
#pragma unroll
            for (int j = 0; j < TG * KSTEPS; ++j) {
                const int rr = RPI * j + lane / LPR;
                const uint4 v = *reinterpret_cast<const uint4 *>(x + (size_t)min(tok0 + rr, S - 1) * M + wave * (M >> 2) + cb);
                a[j / KSTEPS][j % KSTEPS] = v;
            }
        }
#pragma unroll
        for (int i = 0; i < KSTEPS; ++i) {
            const int sc = min(s0 + i, nsteps - 1);
            if constexpr (!STAGE) {
#pragma unroll
                for (int tg = 0; tg < TG; ++tg) a[tg][i] = *reinterpret_cast<const uint4 *>(xp[tg] + sc * 32);
            }
            if constexpr (W_AHEAD) {
#pragma unroll
                for (int g = 0; g < EG; ++g) {
                    const float *wp = wg + (size_t)min(g * 16 + r16, E - 1) * M + kbase + sc * 32;
                    wa[i][g][0] = *reinterpret_cast<const float4 *>(wp);
                    wa[i][g][1] = *reinterpret_cast<const float4 *>(wp + 4);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);       // or the scheduler moves each load down to its use again
        if constexpr (STAGE) {
            char *mine = s_all + wave * (16 * TG * RS);
#pragma unroll
            for (int j = 0; j < TG * KSTEPS; ++j)
                *reinterpret_cast<uint4 *>(mine + (RPI * j + lane / LPR) * RS + (lane % LPR) * 16) = a[j / KSTEPS][j % KSTEPS];
            // (written and read by this wave only: program order is enough)
#pragma unroll
            for (int i = 0; i < KSTEPS; ++i)
#pragma unroll
                for (int tg = 0; tg < TG; ++tg)
                    a[tg][i] = *reinterpret_cast<const uint4 *>(mine + (16 * tg + r16) * RS + i * 64 + kq * 16);
        }
#pragma unroll
        for (int i = 0; i < KSTEPS; ++i) {
            // (no branch here, so that the round stays one block of code and its loads stay ahead of it: a step
            // past the end multiplies zeros)
            const uint32_t keep = s0 + i < nsteps ? 0xffffffffu : 0u;
#pragma unroll
            for (int tg = 0; tg < TG; ++tg)
                a[tg][i] = make_uint4(a[tg][i].x & keep, a[tg][i].y & keep, a[tg][i].z & keep, a[tg][i].w & keep);
#pragma unroll
            for (int g = 0; g < EG; ++g) {
                float4 w0, w1;
                if constexpr (W_AHEAD) {
                    w0 = wa[i][g][0];
                    w1 = wa[i][g][1];
                } else {
                    const float *wp = wg + (size_t)min(g * 16 + r16, E - 1) * M + kbase + min(s0 + i, nsteps - 1) * 32;
                    w0 = *reinterpret_cast<const float4 *>(wp);
                    w1 = *reinterpret_cast<const float4 *>(wp + 4);
                }
                const gate_bf16x8 b = {(bf16_t)w0.x, (bf16_t)w0.y, (bf16_t)w0.z, (bf16_t)w0.w,
                                       (bf16_t)w1.x, (bf16_t)w1.y, (bf16_t)w1.z, (bf16_t)w1.w};
#pragma unroll
                for (int tg = 0; tg < TG; ++tg)
                    acc[tg][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(gate_bf16x8, a[tg][i]), b, acc[tg][g], 0, 0, 0);
            }
        }
    }
    // acc[tg][g][r] = partial logit of token 16 tg + 4 kq + r, expert 16 g + r16
    if constexpr (STAGE) __syncthreads();         // the partial sums take the place of the staged rows
#pragma unroll
    for (int tg = 0; tg < TG; ++tg)
#pragma unroll
        for (int g = 0; g < EG; ++g)
#pragma unroll
            for (int r = 0; r < 4; ++r) part[wave][16 * tg + 4 * kq + r][g * 16 + r16] = acc[tg][g][r];
    __syncthreads();
    const int j = threadIdx.x & 15;               // 16 lanes per token
    constexpr int BT = 16 * TG;
    // routing: [k][BT] experts and raw gate values, four histograms, four rows of column sums - behind the staging area
    int *s_idx = reinterpret_cast<int *>(s_dyn + STAGE_BYTES);
    float *s_graw = reinterpret_cast<float *>(s_idx + (ROUTE ? rt.k : 0) * BT);
    int *s_hist = reinterpret_cast<int *>(s_graw + (ROUTE ? rt.k : 0) * BT);
    float *s_col = reinterpret_cast<float *>(s_hist + 4 * E);
    float colacc[EG];
#pragma unroll
    for (int g = 0; g < EG; ++g) colacc[g] = 0.f;
#pragma unroll
    for (int tg = 0; tg < TG; ++tg) {
        const int t = 16 * tg + (threadIdx.x >> 4);
        const int token = tok0 + t;
        float v[EG];
        float mx = -INFINITY;
#pragma unroll
        for (int g = 0; g < EG; ++g) {
            const int e = g * 16 + j;
            v[g] = e < E ? part[0][t][e] + part[1][t][e] + part[2][t][e] + part[3][t][e] + (bias ? bias[e] : 0.f) : -INFINITY;
            mx = fmaxf(mx, v[g]);
        }
        for (int m = 8; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, WAVE));
        float sum = 0.f;
#pragma unroll
        for (int g = 0; g < EG; ++g) {
            v[g] = g * 16 + j < E ? expf(v[g] - mx) : 0.f;
            sum += v[g];
        }
        for (int m = 8; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, WAVE);
#pragma unroll
        for (int g = 0; g < EG; ++g) {
            const int e = g * 16 + j;
            v[g] = v[g] / sum;
            if (token < S && e < E) scores[(size_t)token * E + e] = v[g];
        }
        if constexpr (ROUTE) {
            // the k rounds of route_topk_kernel on the token's scores (the same keys, the same tie rule)
            uint32_t key[EG];
#pragma unroll
            for (int g = 0; g < EG; ++g) {
                const bool ok = token < S && g * 16 + j < E;
                const float sv = __uint_as_float(__float_as_uint(v[g]) & (ok ? 0xffffffffu : 0u));
                colacc[g] += sv;
                key[g] = ok ? topk_key(sv) : 0u;
            }
            for (int c = 0; c < rt.k; ++c) {
                uint32_t best = key[0];
#pragma unroll
                for (int g = 1; g < EG; ++g) best = max(best, key[g]);
                const uint32_t top = group_reduce(best, 4, [](uint32_t a, uint32_t b2) { return max(a, b2); });
                int cand = INT_MAX;
#pragma unroll
                for (int g = EG - 1; g >= 0; --g)
                    if (key[g] == top) cand = j + (g << 4);                // ends on the lane's lowest such expert
                if (top == 0u) cand = INT_MAX;                             // nothing available (a token past the end)
                const int bi = group_reduce(cand, 4, [](int a, int b2) { return min(a, b2); });
                const bool mine = bi != INT_MAX && (bi & 15) == j;
#pragma unroll
                for (int g = 0; g < EG; ++g)
                    if (mine && (bi >> 4) == g) key[g] = 0u;
                if (j == 0 && token < S) {
                    s_idx[c * BT + t] = bi;
                    s_graw[c * BT + t] = topk_unkey(top);
                }
            }
        }
    }
    if constexpr (ROUTE) {
        // column sums of the scores: fold the wave's four token groups, then (in the tail) the four waves
#pragma unroll
        for (int g = 0; g < EG; ++g) {
            float c = colacc[g];
            c += __shfl_xor(c, 16, WAVE);
            c += __shfl_xor(c, 32, WAVE);
            const int e = g * 16 + j;
            if (lane < 16 && e < E) s_col[wave * E + e] = c;
        }
        topk_block_tail(BT, S, E, rt.k, rt.normalize, s_idx, s_graw, s_hist, s_col, rt.idx, rt.lrank, rt.gates, rt.hist,
                        rt.colsum, rt.nb);
    }
}

}  // namespace mole

#define MOLE_VPL_DISPATCH(vpl, KERNEL, grid, st, ...)                                              \
    do {                                                                                           \
        if ((vpl) <= 1) hipLaunchKernelGGL(KERNEL<1>, grid, dim3(256), 0, st, __VA_ARGS__);         \
        else if ((vpl) <= 2) hipLaunchKernelGGL(KERNEL<2>, grid, dim3(256), 0, st, __VA_ARGS__);    \
        else if ((vpl) <= 4) hipLaunchKernelGGL(KERNEL<4>, grid, dim3(256), 0, st, __VA_ARGS__);    \
        else if ((vpl) <= 8) hipLaunchKernelGGL(KERNEL<8>, grid, dim3(256), 0, st, __VA_ARGS__);    \
        else hipLaunchKernelGGL(KERNEL<16>, grid, dim3(256), 0, st, __VA_ARGS__);                   \
    } while (0)

extern "C" int mole_softmax_fwd(const float *logits, const float *logit_bias, int S, int E, float *scores,
                                mole_stream_t stream) {
    MOLE_REQUIRE(S >= 0 && E >= 1 && E <= MOLE_MAX_EXPERTS, "mole_softmax_fwd: bad sizes S=%d E=%d", S, E);
    if (S == 0) return 0;
    MOLE_REQUIRE(logits && scores, "mole_softmax_fwd: null pointer");
    int logG = 0;
    while ((1 << logG) < E && logG < 6) ++logG;       // (16-lane groups as in the top-k: 18.1 against 17.1 us at 256 experts)
    const int vpl = ceil_div(E, 1 << logG);
    const int tpw = 64 >> logG;
    const dim3 grid(ceil_div(S, 4 * tpw));
    ScopedTiming timing(MOLE_K_GATE_FWD, (hipStream_t)stream);
    MOLE_VPL_DISPATCH(vpl, softmax_fwd_kernel, grid, (hipStream_t)stream, logits, logit_bias, S, E, logG, scores);
    MOLE_LAUNCH_CHECK();
    return 0;
}

// dynamic LDS of gate_fwd_kernel<1, 4, 2, true>: the staged token rows (four waves x 32 rows of 4 x 64 + 16 bytes)
static constexpr unsigned GATE_STAGE_LDS = 4 * 32 * (4 * 64 + 16);
// tokens per block of the fused gate + routing kernels (TG = 2)
static constexpr int GATE_ROUTE_TOKENS = 32;

extern "C" size_t mole_gate_route_workspace_bytes(int S, int E, int k) {
    if (S < 0 || E <= 0 || k <= 0) return 0;
    const size_t nb = (size_t)ceil_div(S > 0 ? S : 1, GATE_ROUTE_TOKENS);
    return align256(nb * k * E * sizeof(int32_t)) + align256((size_t)k * E * sizeof(int32_t)) +
           align256(nb * E * sizeof(float)) + align256((size_t)COLSUM_SLICES * E * sizeof(float));
}

extern "C" int mole_gate_route(const void *x, int dtype, const float *wg, const float *logit_bias, int S, int E, int M,
                               int k, double capacity_factor, int normalize_gate, int alignment, int layout, float *scores,
                               int32_t *idx, int32_t *loc, float *gates, int32_t *row, int32_t *counts,
                               int32_t *kept_rows, int32_t *offsets, int32_t *capacity, float *l_aux, void *workspace,
                               size_t workspace_bytes, mole_stream_t stream) {
    MOLE_REQUIRE(dtype == MOLE_BF16 && S >= 1 && E >= 1 && E <= 64 && M >= 128 && M % 128 == 0,
                 "mole_gate_route: needs bf16 tokens, M a multiple of 128 and at most 64 experts (S=%d E=%d M=%d dtype=%d); "
                 "other shapes: mole_gate_fwd (or mole_gemm_nt + mole_softmax_fwd), then mole_route", S, E, M, dtype);
    MOLE_REQUIRE(k >= 1 && k <= MOLE_MAX_TOPK && k <= E, "mole_gate_route: need 1 <= k <= min(E, %d) (k=%d E=%d)", MOLE_MAX_TOPK, k, E);
    MOLE_REQUIRE(alignment >= 1, "mole_gate_route: alignment must be >= 1");
    MOLE_REQUIRE(layout == MOLE_LAYOUT_PADDED || layout == MOLE_LAYOUT_RAGGED, "mole_gate_route: bad layout %d", layout);
    MOLE_REQUIRE(x && wg && scores && idx && loc && gates && row && counts && kept_rows && offsets && capacity && workspace,
                 "mole_gate_route: null pointer");
    MOLE_REQUIRE((long long)S * k < INT_MAX, "mole_gate_route: S*k too large");
    if (workspace_bytes < mole_gate_route_workspace_bytes(S, E, k)) {
        set_error("mole_gate_route: workspace of %zu bytes, need %zu", workspace_bytes, mole_gate_route_workspace_bytes(S, E, k));
        return MOLE_E_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    const int nb = ceil_div(S, GATE_ROUTE_TOKENS);
    char *ws = (char *)workspace;
    int32_t *hist = (int32_t *)ws;
    ws += align256((size_t)nb * k * E * sizeof(int32_t));
    int32_t *basej = (int32_t *)ws;
    ws += align256((size_t)k * E * sizeof(int32_t));
    float *colsum = (float *)ws;
    ws += align256((size_t)nb * E * sizeof(float));
    float *colpart = (float *)ws;
    const GateRoute rt{k, normalize_gate, nb, idx, loc, hist, gates, colsum};
    const unsigned route_lds = (unsigned)((size_t)k * GATE_ROUTE_TOKENS * 8 + (size_t)E * 4 * 4 * 2);
    const bf16_t *xb = (const bf16_t *)x;
    if (E <= 16)
        timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<1, 4, 2, true, true>, dim3(nb), dim3(256), GATE_STAGE_LDS + route_lds, st, xb, wg,
                     logit_bias, S, E, M, scores, rt);
    else if (E <= 32)
        timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<2, 4, 2, false, true>, dim3(nb), dim3(256), route_lds, st, xb, wg, logit_bias, S,
                     E, M, scores, rt);
    else
        timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<4, 4, 2, false, true>, dim3(nb), dim3(256), route_lds, st, xb, wg, logit_bias, S,
                     E, M, scores, rt);
    MOLE_LAUNCH_CHECK();
    ScopedTiming timing(MOLE_K_ROUTE, st);
    return route_after_topk(hist, basej, colsum, colpart, nb, GATE_ROUTE_TOKENS, S, E, k, capacity_factor, alignment, layout, idx,
                            loc, row, counts, kept_rows, offsets, capacity, l_aux, st);
}

extern "C" int mole_gate_fwd(const void *x, int dtype, const float *wg, const float *logit_bias, int S, int E, int M,
                             float *scores, mole_stream_t stream) {
    MOLE_REQUIRE(S >= 0 && E >= 1 &&
                     ((dtype == MOLE_BF16 && E <= 256 && M >= 128 && M % 128 == 0) || (dtype == MOLE_F32 && E <= 32 && M >= 4 && M % 4 == 0)),
                 "mole_gate_fwd: needs bf16 tokens with M a multiple of 128 and at most 256 experts, or fp32 tokens with M a "
                 "multiple of 4 and at most 32 experts (S=%d E=%d M=%d dtype=%d)", S, E, M, dtype);
    if (S == 0) return 0;
    MOLE_REQUIRE(x && wg && scores, "mole_gate_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MOLE_F32) {
        MOLE_REQUIRE((((uintptr_t)x | (uintptr_t)wg) & 15) == 0, "mole_gate_fwd: x and wg must be 16-byte aligned");
        const dim3 grid4(ceil_div(S, 4));
        const float *xf = (const float *)x;
        if (E <= 8) timed_launch(MOLE_K_GATE_FWD, gate_fwd_f32_kernel<8>, grid4, dim3(256), 0, st, xf, wg, logit_bias, S, E, M, scores);
        else if (E <= 16) timed_launch(MOLE_K_GATE_FWD, gate_fwd_f32_kernel<16>, grid4, dim3(256), 0, st, xf, wg, logit_bias, S, E, M, scores);
        else timed_launch(MOLE_K_GATE_FWD, gate_fwd_f32_kernel<32>, grid4, dim3(256), 0, st, xf, wg, logit_bias, S, E, M, scores);
        MOLE_LAUNCH_CHECK();
        return 0;
    }
    const bf16_t *xb = (const bf16_t *)x;
    const int eg = ceil_div(E, 16);
    // small gates: 32 tokens per block (Wg, which every block reads in full, is then read half as often)
    const dim3 grid(ceil_div(S, eg <= 2 ? 32 : 16));
    // (16 experts or fewer: staged, 34 KB of LDS; 10.6 against 11.6 us straight from memory at 16384 x 1024, and 11.1
    // with the whole quarter row in one round of eight steps)
    const GateRoute none{};
    if (eg == 1) timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<1, 4, 2, true>, grid, dim3(256), GATE_STAGE_LDS, st, xb, wg, logit_bias, S, E, M, scores, none);
    else if (eg == 2) timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<2, 4, 2, false>, grid, dim3(256), 0, st, xb, wg, logit_bias, S, E, M, scores, none);
    // (33-64 experts: Wg is 4 times as large, so more tokens share a block's pass over it: 8192 x 2048 x 64: 35.6 us
    // with 16 tokens per block, 22.5 with 32, 27.7 with 64 (128 blocks); 16384 x 1024 x 64: 35.5 / 23.6 / 18.5 us)
    else if (eg <= 4 && S >= 64 * 256) timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<4, 4, 4, false>, dim3(ceil_div(S, 64)), dim3(256), 0, st, xb, wg, logit_bias, S, E, M, scores, none);
    else if (eg <= 4 && S >= 32 * 128) timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<4, 4, 2, false>, dim3(ceil_div(S, 32)), dim3(256), 0, st, xb, wg, logit_bias, S, E, M, scores, none);
    else if (eg <= 4) timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<4, 4, 1, false>, grid, dim3(256), 0, st, xb, wg, logit_bias, S, E, M, scores, none);
    else if (eg <= 8) timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<8, 4, 1, false>, grid, dim3(256), 0, st, xb, wg, logit_bias, S, E, M, scores, none);
    else timed_launch(MOLE_K_GATE_FWD, gate_fwd_kernel<16, 2, 1, false>, grid, dim3(256), 0, st, xb, wg, logit_bias, S, E, M, scores, none);
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" int mole_softmax_bwd(const float *dscores, const float *scores, int S, int E, float *dlogits,
                                mole_stream_t stream) {
    MOLE_REQUIRE(S >= 0 && E >= 1 && E <= MOLE_MAX_EXPERTS, "mole_softmax_bwd: bad sizes S=%d E=%d", S, E);
    if (S == 0) return 0;
    MOLE_REQUIRE(dscores && scores && dlogits, "mole_softmax_bwd: null pointer");
    int logG = 0;
    while ((1 << logG) < E && logG < 6) ++logG;
    const int vpl = ceil_div(E, 1 << logG);
    const int tpw = 64 >> logG;
    const dim3 grid(ceil_div(S, 4 * tpw));
    ScopedTiming timing(MOLE_K_GATE_BWD, (hipStream_t)stream);
    MOLE_VPL_DISPATCH(vpl, softmax_bwd_kernel, grid, (hipStream_t)stream, dscores, scores, S, E, logG, dlogits);
    MOLE_LAUNCH_CHECK();
    return 0;
}

extern "C" int mole_gate_bwd(const float *dgates, const float *scores, const int32_t *idx, int S, int E, int k,
                             int normalize_gate, int through_softmax, const int32_t *counts0, const float *d_l_aux,
                             float *dlogits, mole_stream_t stream) {
    MOLE_REQUIRE(S >= 0 && E >= 1 && E <= MOLE_MAX_EXPERTS && k >= 1 && k <= MOLE_MAX_TOPK && k <= E,
                 "mole_gate_bwd: bad sizes S=%d E=%d k=%d", S, E, k);
    if (S == 0) return 0;
    MOLE_REQUIRE(dgates && scores && idx && dlogits, "mole_gate_bwd: null pointer");
    MOLE_REQUIRE((counts0 == nullptr) == (d_l_aux == nullptr), "mole_gate_bwd: counts0 and d_l_aux go together");
    int logG = 0;
    while ((1 << logG) < E && logG < 6) ++logG;
    const int vpl = ceil_div(E, 1 << logG);
    const int tpw = 64 >> logG;
    const dim3 grid(ceil_div(S, 4 * tpw));
    ScopedTiming timing(MOLE_K_GATE_BWD, (hipStream_t)stream);
    MOLE_VPL_DISPATCH(vpl, gate_bwd_kernel, grid, (hipStream_t)stream, dgates, scores, idx, S, E, k, logG,
                      normalize_gate, through_softmax, counts0, d_l_aux, dlogits);
    MOLE_LAUNCH_CHECK();
    return 0;
}
