// Grouped expert FFN on MFMA tiles: forward and backward of
//     h = xd.w1^T + b1 ;  a = gelu_erf(h) ;  out = a.w2 + b2
// with bias, GELU and GELU' fused into the GEMM epilogues.
//
// Replaces _BatchRecord::bffn_fwd / bffn_bwd / bffn_bwd_acc (MOLE/cpp/core.cpp:344-356, 381-414,
// 457-491: baddbmm, gelu, matmul, sum) and the separate GELU-backward kernel (MOLE/cpp/gelu.cu:3-58).
//
// One kernel template covers the six products.  A block of 256 threads (4 waves, 2x2) owns a
// BM x BN tile of the output and walks K in steps of 128 bytes (64 bf16 / 32 fp32).  Operands are
// staged global -> registers -> LDS as 16-byte chunks; the LDS image is always [row][k] with the
// chunk index XOR-swizzled by the row, so the MFMA fragment reads are conflict-free 16-byte reads
// whatever the operand's layout in HBM was.  An operand that is K-strided in HBM (w2 in the
// forward, both operands of the weight gradients) is transposed in registers on its way into LDS.
// The next K-step's global loads are issued before the current step's MFMAs; LDS is double
// buffered, one barrier per step.
//
// Row-ragged products (forward, data gradients) take their M extent per expert from
// offsets/kept_rows on the device; a block finds its (expert, m-tile) with a wave-parallel prefix
// search, so no host synchronisation is needed to launch.  Weight gradients contract over the
// expert's rows instead (K extent ragged).
#include "gemm.h"

#include <stdlib.h>

namespace mole {

// ---------------------------------------------------------------------------------------------
// tile geometry shared by both element types: a row of a staged tile is 128 bytes = 8 chunks
// ---------------------------------------------------------------------------------------------
constexpr int GEMM_THREADS = 256;
constexpr int CHUNKS = 8;  // 16-byte chunks per tile row

template <typename T> struct Elem;
template <> struct Elem<bf16_t> { static constexpr int EPC = 8, BK = 64; };
template <> struct Elem<float> { static constexpr int EPC = 4, BK = 32; };

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }
__device__ __forceinline__ int lds_off(int row, int chunk) { return (row * CHUNKS + (chunk ^ swz(row))) * 16; }

// K-contiguous operand: element (r, k) at p[r*ld + k]
template <typename T, int ROWS> struct LoaderKC {
    static constexpr int EPC = Elem<T>::EPC, BK = Elem<T>::BK;
    static constexpr int NCH = ROWS / 32;  // chunks per thread
    uint4 regs[NCH];
    __device__ __forceinline__ void load(const T *p, long ld, int r0, int r_ext, int k0, int K) {
        const int tid = threadIdx.x;
        const int ch = tid & 7;
        const int k = k0 + ch * EPC;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int r = r0 + (tid >> 3) + 32 * i;
            if (r < r_ext && k < K)
                regs[i] = *reinterpret_cast<const uint4 *>(p + (long)r * ld + k);
            else
                regs[i] = make_uint4(0, 0, 0, 0);
        }
    }
    __device__ __forceinline__ void store(char *lds) const {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < NCH; ++i)
            *reinterpret_cast<uint4 *>(lds + lds_off((tid >> 3) + 32 * i, tid & 7)) = regs[i];
    }
};

// K-strided operand: element (r, k) at p[k*ld + r].  A thread owns EPC x EPC blocks (EPC k-rows of
// EPC consecutive r), which it transposes in registers so that LDS again holds [r][k].
template <typename T, int ROWS> struct LoaderKS {
    static constexpr int EPC = Elem<T>::EPC, BK = Elem<T>::BK;
    static constexpr int RB = ROWS / EPC;          // r-blocks per tile
    static constexpr int NBLK = CHUNKS * RB;        // blocks per tile
    static constexpr int NB = (NBLK + GEMM_THREADS - 1) / GEMM_THREADS;
    uint4 regs[NB][EPC];
    __device__ __forceinline__ void load(const T *p, long ld, int r0, int r_ext, int k0, int K) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int bq = tid + GEMM_THREADS * i;
            const int rb = bq % RB, kb = bq / RB;
            const int r = r0 + rb * EPC;
            const bool rok = (NBLK % GEMM_THREADS == 0 || bq < NBLK) && r < r_ext;
#pragma unroll
            for (int kk = 0; kk < EPC; ++kk) {
                const int k = k0 + kb * EPC + kk;
                if (rok && k < K)
                    regs[i][kk] = *reinterpret_cast<const uint4 *>(p + (long)k * ld + r);
                else
                    regs[i][kk] = make_uint4(0, 0, 0, 0);
            }
        }
    }
    __device__ __forceinline__ void store(char *lds) const {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int bq = tid + GEMM_THREADS * i;
            if (NBLK % GEMM_THREADS != 0 && bq >= NBLK) continue;
            const int rb = bq % RB, kb = bq / RB;
            if constexpr (EPC == 4) {  // fp32: 4x4 transpose is a renaming
                const uint4 *q = regs[i];
                const uint4 c0 = make_uint4(q[0].x, q[1].x, q[2].x, q[3].x);
                const uint4 c1 = make_uint4(q[0].y, q[1].y, q[2].y, q[3].y);
                const uint4 c2 = make_uint4(q[0].z, q[1].z, q[2].z, q[3].z);
                const uint4 c3 = make_uint4(q[0].w, q[1].w, q[2].w, q[3].w);
                *reinterpret_cast<uint4 *>(lds + lds_off(rb * 4 + 0, kb)) = c0;
                *reinterpret_cast<uint4 *>(lds + lds_off(rb * 4 + 1, kb)) = c1;
                *reinterpret_cast<uint4 *>(lds + lds_off(rb * 4 + 2, kb)) = c2;
                *reinterpret_cast<uint4 *>(lds + lds_off(rb * 4 + 3, kb)) = c3;
            } else {  // bf16: 8x8 transpose of 16-bit values with byte permutes
                const uint4 *q = regs[i];
                const uint32_t w[8][4] = {{q[0].x, q[0].y, q[0].z, q[0].w}, {q[1].x, q[1].y, q[1].z, q[1].w},
                                          {q[2].x, q[2].y, q[2].z, q[2].w}, {q[3].x, q[3].y, q[3].z, q[3].w},
                                          {q[4].x, q[4].y, q[4].z, q[4].w}, {q[5].x, q[5].y, q[5].z, q[5].w},
                                          {q[6].x, q[6].y, q[6].z, q[6].w}, {q[7].x, q[7].y, q[7].z, q[7].w}};
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const int d = c >> 1;
                    const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
                    uint4 o;
                    o.x = __builtin_amdgcn_perm(w[1][d], w[0][d], sel);
                    o.y = __builtin_amdgcn_perm(w[3][d], w[2][d], sel);
                    o.z = __builtin_amdgcn_perm(w[5][d], w[4][d], sel);
                    o.w = __builtin_amdgcn_perm(w[7][d], w[6][d], sel);
                    *reinterpret_cast<uint4 *>(lds + lds_off(rb * 8 + c, kb)) = o;
                }
            }
        }
    }
};

template <typename T, bool KS, int ROWS> struct LoaderSel { typedef LoaderKC<T, ROWS> type; };
template <typename T, int ROWS> struct LoaderSel<T, true, ROWS> { typedef LoaderKS<T, ROWS> type; };

// one K-step (128 bytes of K) of MFMAs for a wave tile of TM x TN 32x32 blocks
template <typename T, int TM, int TN>
__device__ __forceinline__ void mma_step(const char *ldsA, const char *ldsB, int rowA0, int rowB0,
                                         f32x16 (&acc)[TM][TN]) {
    const int lane = threadIdx.x & 63;
    const int lr = lane & 31, h = lane >> 5;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        uint4 a[TM], b[TN];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
            a[tm] = *reinterpret_cast<const uint4 *>(ldsA + lds_off(rowA0 + tm * 32 + lr, 2 * kk + h));
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
            b[tn] = *reinterpret_cast<const uint4 *>(ldsB + lds_off(rowB0 + tn * 32 + lr, 2 * kk + h));
        if constexpr (sizeof(T) == 2) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, a[tm]), __builtin_bit_cast(bf16x8, b[tn]), acc[tm][tn], 0, 0, 0);
        } else {
            // the four k of a 16-byte fragment, the cells of the wave tile innermost: consecutive MFMAs write
            // different accumulators
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn) {
                        const uint32_t aw[4] = {a[tm].x, a[tm].y, a[tm].z, a[tm].w}, bw[4] = {b[tn].x, b[tn].y, b[tn].z, b[tn].w};
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(aw[j]), __uint_as_float(bw[j]), acc[tm][tn], 0, 0, 0);
                    }
        }
    }
}

// Row-ragged: C[rows_e, N] = A[rows_e, K] . B_e   (A K-contiguous; B_e [N,K] or, B_KS, [K,N])
// Weight gradient (WG): C_e[M, N] = sum_{r in rows_e} A[r, M]^T . B[r, N]  (both K-strided)
template <typename T, bool A_KS, bool B_KS, bool WG, int BM, int BN, int EPI>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_kernel(const GemmArgs g) {
    constexpr int BK = Elem<T>::BK;
    constexpr int TM = BM / 64, TN = BN / 64;  // 2x2 waves, 32x32 MFMA blocks
    extern __shared__ __align__(16) char smem[];
    constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;

    // ---- which tile am I?  Blocks are dealt round-robin to the 8 XCDs (block b runs on XCD b mod 8):
    //      give each XCD a contiguous range of the REAL tiles, so that neighbours share operands in
    //      its L2 and every XCD gets the same share.  For row-ragged products the number of real
    //      tiles is only known here (the grid is sized for the worst case), hence the device-side sum.
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_tiles = (g.N + BN - 1) / BN;
    int e, mt, nt, m_ext, k_ext;
    long row0;  // first row of the expert
    if constexpr (!WG) {
        int total_m_tiles;
        if (g.offsets == nullptr) {
            total_m_tiles = (g.single_rows + BM - 1) / BM;
        } else {
            int part = 0;
            for (int ee = lane; ee < g.E; ee += WAVE) part += (g.kept[ee] + BM - 1) / BM;
            for (int d = WAVE / 2; d >= 1; d >>= 1) part += __shfl_xor(part, d, WAVE);
            total_m_tiles = part;
        }
        const int total = total_m_tiles * n_tiles;
        const int per_xcd = (total + 7) >> 3;
        const int slot = blockIdx.x >> 3;
        const int t = (blockIdx.x & 7) * per_xcd + slot;
        if (slot >= per_xcd || t >= total) return;
        const int mtg = t / n_tiles;
        nt = t % n_tiles;
        if (g.offsets == nullptr) {
            e = 0; mt = mtg; m_ext = g.single_rows; row0 = 0;
        } else {
            int run = 0, found = -1, fmt = 0;
            for (int base = 0; base < g.E && found < 0; base += WAVE) {
                const int ee = base + lane;
                const int tiles = ee < g.E ? (g.kept[ee] + BM - 1) / BM : 0;
                int incl = tiles;
                for (int d = 1; d < WAVE; d <<= 1) {
                    const int y = __shfl_up(incl, d, WAVE);
                    if (lane >= d) incl += y;
                }
                const unsigned long long hit = __ballot(run + incl > mtg);
                if (hit) {
                    const int src = __ffsll(hit) - 1;
                    found = base + src;
                    fmt = mtg - (run + __shfl(incl - tiles, src, WAVE));
                }
                run += __shfl(incl, WAVE - 1, WAVE);
            }
            if (found < 0) return;
            e = found; mt = fmt;
            m_ext = g.kept[e];
            row0 = g.offsets[e];
        }
        k_ext = g.K;
    } else {
        const int nblk = gridDim.x;
        const int t = (blockIdx.x & 7) * (nblk >> 3) + (blockIdx.x >> 3);
        if (t >= g.n_blocks) return;
        const int m_tiles = (g.M + BM - 1) / BM;
        e = t / (m_tiles * n_tiles);
        const int rem = t % (m_tiles * n_tiles);
        mt = rem / n_tiles;
        nt = rem % n_tiles;
        m_ext = g.M;
        k_ext = g.kept ? g.kept[e] : g.single_rows;
        row0 = g.offsets ? g.offsets[e] : 0;
    }
    const int m0 = mt * BM, n0 = nt * BN;

    const T *Ap, *Bp;
    if constexpr (!WG) {
        Ap = (const T *)g.A + row0 * g.lda;           // rows of this expert
        Bp = (const T *)g.B + (long)e * g.strideB;    // this expert's weights
    } else {
        Ap = (const T *)g.A + row0 * g.lda;           // [k = row][M]
        Bp = (const T *)g.B + row0 * g.ldb;           // [k = row][N]
    }

    typename LoaderSel<T, A_KS, BM>::type la;
    typename LoaderSel<T, B_KS, BN>::type lb;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

    const int wm = wave >> 1, wn = wave & 1;
    const int rowA0 = wm * (BM / 2), rowB0 = wn * (BN / 2);
    const int nk = (k_ext + BK - 1) / BK;

    if (nk > 0) {
        la.load(Ap, g.lda, m0, m_ext, 0, k_ext);
        lb.load(Bp, g.ldb, n0, g.N, 0, k_ext);
        la.store(smem);
        lb.store(smem + A_BYTES);
    }
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        char *cur = smem + (kt & 1) * STAGE;
        char *nxt = smem + ((kt + 1) & 1) * STAGE;
        const bool more = kt + 1 < nk;
        if (more) {
            la.load(Ap, g.lda, m0, m_ext, (kt + 1) * BK, k_ext);
            lb.load(Bp, g.ldb, n0, g.N, (kt + 1) * BK, k_ext);
        }
        mma_step<T, TM, TN>(cur, cur + A_BYTES, rowA0, rowB0, acc);
        if (more) {
            la.store(nxt);
            lb.store(nxt + A_BYTES);
        }
        __syncthreads();
    }

    // ---- epilogue.  acc[tm][tn][i] is C[m, n] with n = lane%32 and m = 8*(i/4) + 4*(lane/32) + i%4
    const int lr = lane & 31, h = lane >> 5;
    long crow0;
    char *Cb = (char *)g.C;
    if constexpr (!WG) crow0 = row0; else { crow0 = 0; Cb += (long)e * g.strideC * sizeof(T); }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int n = n0 + rowB0 + tn * 32 + lr;
        if (n >= g.N) continue;
        float bias = 0.f;
        if constexpr (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU) bias = to_f32(((const T *)g.bias)[(long)e * g.N + n]);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            // GELU': the 16 pre-activations of this cell are fetched first, unconditionally (rows past the end read
            // the expert's last row and are not used) - a load behind the row test below would be waited for
            // before the next one is issued
            float hv16[16];
            if constexpr (EPI == EPI_DGELU) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int m = m0 + rowA0 + tm * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                    hv16[i] = to_f32(((const T *)g.H)[(crow0 + min(m, m_ext - 1)) * g.ldc + n]);
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int m = m0 + rowA0 + tm * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                if (m >= m_ext) continue;
                const long off = (crow0 + m) * g.ldc + n;
                float v = acc[tm][tn][i];
                if constexpr (EPI == EPI_F32) {
                    ((float *)g.C)[off] = v;
                } else if constexpr (EPI == EPI_STORE) {
                    ((T *)Cb)[off] = from_f32<T>(v);
                } else if constexpr (EPI == EPI_BIAS) {
                    ((T *)Cb)[off] = from_f32<T>(v + bias);
                } else if constexpr (EPI == EPI_BIAS_GELU) {
                    v += bias;
                    ((T *)Cb)[off] = from_f32<T>(v);
                    ((T *)g.C2)[off] = from_f32<T>(gelu_erf(v));
                } else if constexpr (EPI == EPI_DGELU) {
                    const float hv = hv16[i];
                    const float d = g.gelu_bwd == MOLE_GELU_BWD_TANH ? d_gelu_tanh(hv) : d_gelu_exact(hv);
                    ((T *)Cb)[off] = from_f32<T>(v * d);
                } else {  // EPI_WGRAD
                    if (g.accumulate) v += to_f32(((T *)Cb)[off]);
                    ((T *)Cb)[off] = from_f32<T>(v);
                }
            }
        }
    }
}

// column sums over an expert's rows: out[e, n] (+)= sum_{r in rows_e} in[r, n]
// (torch::sum_out(g_b2, go, {1}) / (g_b1, t, {1}), MOLE/cpp/core.cpp:399, 408).
// Both sums run in one launch: blocks [0, nbx0) of a grid row take the first matrix, the rest the
// second, so the narrow one (M columns) does not leave most of the chip idle on its own.
// A block of 16 waves owns 64*VEC columns of one expert; wave w sums rows w, w+16, ... with 8-byte
// loads per lane (8 rows in flight), then the 16 partial rows are folded through LDS in a fixed order.
constexpr int BG_WAVES = 16;
constexpr int BG_FLY = 8;
template <typename T>
__device__ __forceinline__ void bias_acc(float *acc, uint2 v) {
    if constexpr (sizeof(T) == 2) {
        acc[0] += __uint_as_float(v.x << 16); acc[1] += __uint_as_float(v.x & 0xffff0000u);
        acc[2] += __uint_as_float(v.y << 16); acc[3] += __uint_as_float(v.y & 0xffff0000u);
    } else {
        acc[0] += __uint_as_float(v.x); acc[1] += __uint_as_float(v.y);
    }
}
template <typename T>
__global__ __launch_bounds__(BG_WAVES * 64) void bias_grad_kernel(const T *__restrict__ in0, int N0, T *__restrict__ out0,
                                                                   int nbx0, const T *__restrict__ in1, int N1,
                                                                   T *__restrict__ out1,
                                                                   const int32_t *__restrict__ offsets,
                                                                   const int32_t *__restrict__ kept, int accumulate) {
    constexpr int VEC = 8 / sizeof(T);   // elements per 8-byte load: 4 bf16 or 2 fp32
    __shared__ float s_part[BG_WAVES][64 * VEC];
    const bool first = (int)blockIdx.x < nbx0;
    const T *__restrict__ in = first ? in0 : in1;
    T *__restrict__ out = first ? out0 : out1;
    const int N = first ? N0 : N1;
    const int bx = first ? blockIdx.x : blockIdx.x - nbx0;
    const int e = blockIdx.y;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int n = (bx * 64 + lane) * VEC;
    const long r0 = offsets[e];
    const int rows = kept[e];
    float acc[VEC];
#pragma unroll
    for (int q = 0; q < VEC; ++q) acc[q] = 0.f;
    if (n < N) {
        const T *p = in + r0 * (long)N + n;
        int r = w;
        for (; r + (BG_FLY - 1) * BG_WAVES < rows; r += BG_FLY * BG_WAVES) {
            uint2 v[BG_FLY];
#pragma unroll
            for (int u = 0; u < BG_FLY; ++u) v[u] = *reinterpret_cast<const uint2 *>(p + (long)(r + u * BG_WAVES) * N);
#pragma unroll
            for (int u = 0; u < BG_FLY; ++u) bias_acc<T>(acc, v[u]);
        }
        for (; r < rows; r += BG_WAVES) bias_acc<T>(acc, *reinterpret_cast<const uint2 *>(p + (long)r * N));
    }
#pragma unroll
    for (int q = 0; q < VEC; ++q) s_part[w][lane * VEC + q] = acc[q];
    __syncthreads();
    for (int c = threadIdx.x; c < 64 * VEC; c += BG_WAVES * 64) {
        const int nn = bx * 64 * VEC + c;
        if (nn >= N) continue;
        float v = 0.f;
#pragma unroll
        for (int ww = 0; ww < BG_WAVES; ++ww) v += s_part[ww][c];
        if (accumulate) v += to_f32(out[(long)e * N + nn]);
        out[(long)e * N + nn] = from_f32<T>(v);
    }
}

template <typename T, bool A_KS, bool B_KS, bool WG, int BM, int BN, int EPI>
static int launch_gemm(GemmArgs g, int tiles, hipStream_t st, int kid) {
    if (tiles <= 0) return 0;
    g.n_blocks = tiles;
    const int grid = (tiles + 7) & ~7;
    const size_t lds = 2 * (size_t)(BM + BN) * 128;
    auto kern = gemm_kernel<T, A_KS, B_KS, WG, BM, BN, EPI>;
    static bool attr_done = false;  // per instantiation
    if (!attr_done && lds > 64 * 1024) {
        MOLE_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_done = true;
    }
    timed_launch(kid, kern, dim3(grid), dim3(GEMM_THREADS), (unsigned)lds, st, g);
    MOLE_LAUNCH_CHECK();
    return 0;
}

constexpr int TBM = 128, TBN = 128;  // tile of the generic kernel

// A -DMOLE_TUNING build reads MOLE_GEMM=generic from the environment, which sends every product to the generic kernel
// (for A/B runs against the direct-to-LDS kernels).
static bool fast_path_enabled() {
#ifdef MOLE_TUNING
    static const bool on = [] {
        const char *v = getenv("MOLE_GEMM");
        return !(v && v[0] == 'g');
    }();
    return on;
#else
    return true;
#endif
}

// products go to the direct-to-LDS kernel of their element type when their shape allows it
template <typename T, bool A_KS, bool B_KS, bool WG, int EPI>
static int run_gemm(const GemmArgs &g, int max_rows, int tiles_generic, hipStream_t st, int kid) {
    if constexpr (sizeof(T) == 2) {
        if (fast_path_enabled()) {
            const int rc = launch_gemm256(g, A_KS, B_KS, WG, EPI, max_rows, st, kid);
            if (rc != -100) return rc;
        }
    } else {
        if (fast_path_enabled()) {
            const int rc = launch_gemm_f32(g, A_KS, B_KS, WG, EPI, max_rows, st, kid);
            if (rc != -100) return rc;
        }
    }
    // only the direct-to-LDS kernels sum an operand on the side: the caller asks gemm*_sums_operand() first
    MOLE_REQUIRE(g.colsum == nullptr, "grouped GEMM: operand sums requested from a kernel that does not produce them");
    return launch_gemm<T, A_KS, B_KS, WG, TBM, TBN, EPI>(g, tiles_generic, st, kid);
}


template <typename T>
static int ffn_fwd_t(const void *xd, const int32_t *offsets, const int32_t *kept, int E, int max_rows, int M, int F,
                     const void *w1, const void *b1, const void *w2, const void *b2, void *h, void *a, void *out,
                     hipStream_t st) {
    const int m_tiles = max_rows / TBM + E;  // every expert may end in a partial tile
    GemmArgs g{};
    g.offsets = offsets; g.kept = kept; g.E = E; g.m_tiles_bound = m_tiles;
    // h = xd . w1^T + b1, a = gelu(h)
    g.A = xd; g.lda = M; g.B = w1; g.ldb = M; g.strideB = (long)F * M; g.N = F; g.K = M;
    g.C = h; g.C2 = a; g.ldc = F; g.bias = b1;
    if (int rc = run_gemm<T, false, false, false, EPI_BIAS_GELU>(g, max_rows, m_tiles * ceil_div(F, TBN), st, MOLE_K_FFN_FWD1)) return rc;
    // out = a . w2 + b2   (w2 [F,M]: K-strided)
    g.A = a; g.lda = F; g.B = w2; g.ldb = M; g.strideB = (long)F * M; g.N = M; g.K = F;
    g.C = out; g.C2 = nullptr; g.ldc = M; g.bias = b2;
    return run_gemm<T, false, true, false, EPI_BIAS>(g, max_rows, m_tiles * ceil_div(M, TBN), st, MOLE_K_FFN_FWD2);
}

template <typename T>
static int ffn_bwd_t(const void *go, const void *xd, const void *h, const void *a, const int32_t *offsets,
                     const int32_t *kept, int E, int max_rows, int M, int F, const void *w1, const void *w2, void *t,
                     void *g_w1, void *g_b1, void *g_w2, void *g_b2, void *gx, int accumulate, int gelu_bwd,
                     hipStream_t st) {
    const int m_tiles = max_rows / TBM + E;
    GemmArgs g{};
    g.offsets = offsets; g.kept = kept; g.E = E; g.m_tiles_bound = m_tiles;
    g.accumulate = accumulate; g.gelu_bwd = gelu_bwd;
    const int wg_tiles = E * ceil_div(F, TBM) * ceil_div(M, TBN);
    // The bias gradients are sums of go and of t over every expert's rows: go and t are operands of the two
    // weight-gradient products, whose direct-to-LDS kernels sum an operand on the side in the blocks that see the
    // whole operand (bf16: one more MFMA against a block of ones; fp32: the fragments are added up as they pass).
    // The generic kernel leaves them to bias_grad_kernel.
    GemmArgs gw2{};
    gw2 = g;
    gw2.A = a; gw2.lda = F; gw2.B = go; gw2.ldb = M; gw2.M = F; gw2.N = M; gw2.C = g_w2; gw2.ldc = M; gw2.strideC = (long)F * M;
    bool fused_sums = false;
    if constexpr (sizeof(T) == 2)
        fused_sums = fast_path_enabled() && gemm256_sums_operand(gw2, MOLE_K_FFN_GW2) && gemm256_sums_operand(gw2, MOLE_K_FFN_GW1);
    else
        fused_sums = fast_path_enabled() && gemm_f32_sums_operand(gw2);
    // g_w2[e] = a^T . go          (contract over the expert's rows); g_b2 = sum go
    if (fused_sums) { gw2.colsum = g_b2; gw2.colsum_side = 2; }
    if (int rc = run_gemm<T, true, true, true, EPI_WGRAD>(gw2, max_rows, wg_tiles, st, MOLE_K_FFN_GW2)) return rc;
    // t = (go . w2^T) * gelu'(h)   (w2 [F,M]: K = M contiguous)
    g.A = go; g.lda = M; g.B = w2; g.ldb = M; g.strideB = (long)F * M; g.N = F; g.K = M; g.C = t; g.ldc = F; g.H = h;
    if (int rc = run_gemm<T, false, false, false, EPI_DGELU>(g, max_rows, m_tiles * ceil_div(F, TBN), st, MOLE_K_FFN_DA)) return rc;
    if (!fused_sums) {
        // g_b2 = sum go ; g_b1 = sum t
        ScopedTiming timing(MOLE_K_FFN_GB, st);
        const int cols_per_block = 512 / (int)sizeof(T);
        const int nb2 = ceil_div(M, cols_per_block), nb1 = ceil_div(F, cols_per_block);
        hipLaunchKernelGGL(bias_grad_kernel<T>, dim3(nb2 + nb1, E), dim3(BG_WAVES * 64), 0, st, (const T *)go, M, (T *)g_b2, nb2,
                           (const T *)t, F, (T *)g_b1, offsets, kept, accumulate);
        MOLE_LAUNCH_CHECK();
    }
    // g_w1[e] = t^T . xd ; g_b1 = sum t
    g.A = t; g.lda = F; g.B = xd; g.ldb = M; g.M = F; g.N = M; g.C = g_w1; g.ldc = M; g.strideC = (long)F * M;
    if (fused_sums) { g.colsum = g_b1; g.colsum_side = 1; }
    if (int rc = run_gemm<T, true, true, true, EPI_WGRAD>(g, max_rows, wg_tiles, st, MOLE_K_FFN_GW1)) return rc;
    g.colsum = nullptr; g.colsum_side = 0;
    // gx = t . w1                  (w1 [F,M]: K = F strided)
    if (gx != nullptr) {
        g.A = t; g.lda = F; g.B = w1; g.ldb = M; g.strideB = (long)F * M; g.N = M; g.K = F; g.C = gx; g.ldc = M;
        if (int rc = run_gemm<T, false, true, false, EPI_STORE>(g, max_rows, m_tiles * ceil_div(M, TBN), st, MOLE_K_FFN_GX)) return rc;
    }
    return 0;
}

static int check_ffn(const char *fn, int dtype, int E, int max_rows, int M, int F) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "%s: bad dtype %d", fn, dtype);
    const int epc = dtype == MOLE_BF16 ? 8 : 4;
    MOLE_REQUIRE(E >= 1 && max_rows >= 0 && M > 0 && F > 0, "%s: bad sizes E=%d max_rows=%d M=%d F=%d", fn, E, max_rows, M, F);
    MOLE_REQUIRE(M % epc == 0 && F % epc == 0, "%s: M=%d and F=%d must be multiples of %d", fn, M, F, epc);
    return 0;
}
static bool al16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace mole

using namespace mole;

extern "C" int mole_ffn_fwd(const void *xd, int dtype, const int32_t *offsets, const int32_t *kept_rows, int E,
                            int max_rows, int M, int F, const void *w1, const void *b1, const void *w2, const void *b2,
                            void *h, void *a, void *out, mole_stream_t stream) {
    if (int rc = check_ffn("mole_ffn_fwd", dtype, E, max_rows, M, F)) return rc;
    if (max_rows == 0) return 0;
    MOLE_REQUIRE(xd && offsets && kept_rows && w1 && b1 && w2 && b2 && h && a && out, "mole_ffn_fwd: null pointer");
    MOLE_REQUIRE(al16(xd) && al16(w1) && al16(w2) && al16(h) && al16(a) && al16(out), "mole_ffn_fwd: buffers must be 16-byte aligned");
    if (dtype == MOLE_BF16)
        return ffn_fwd_t<bf16_t>(xd, offsets, kept_rows, E, max_rows, M, F, w1, b1, w2, b2, h, a, out, (hipStream_t)stream);
    return ffn_fwd_t<float>(xd, offsets, kept_rows, E, max_rows, M, F, w1, b1, w2, b2, h, a, out, (hipStream_t)stream);
}

extern "C" int mole_ffn_bwd(const void *go, const void *xd, const void *h, const void *a, int dtype,
                            const int32_t *offsets, const int32_t *kept_rows, int E, int max_rows, int M, int F,
                            const void *w1, const void *w2, void *t, void *g_w1, void *g_b1, void *g_w2, void *g_b2,
                            void *gx, int accumulate, int gelu_bwd, mole_stream_t stream) {
    if (int rc = check_ffn("mole_ffn_bwd", dtype, E, max_rows, M, F)) return rc;
    MOLE_REQUIRE(gelu_bwd == MOLE_GELU_BWD_TANH || gelu_bwd == MOLE_GELU_BWD_EXACT, "mole_ffn_bwd: bad gelu_bwd %d", gelu_bwd);
    MOLE_REQUIRE(offsets && kept_rows && w1 && w2 && g_w1 && g_b1 && g_w2 && g_b2, "mole_ffn_bwd: null pointer");
    MOLE_REQUIRE(max_rows == 0 || (go && xd && h && a && t), "mole_ffn_bwd: null activation pointer");
    MOLE_REQUIRE(al16(go) && al16(xd) && al16(h) && al16(a) && al16(t) && al16(w1) && al16(w2) && al16(gx),
                 "mole_ffn_bwd: buffers must be 16-byte aligned");
    if (dtype == MOLE_BF16)
        return ffn_bwd_t<bf16_t>(go, xd, h, a, offsets, kept_rows, E, max_rows, M, F, w1, w2, t, g_w1, g_b1, g_w2, g_b2,
                                 gx, accumulate, gelu_bwd, (hipStream_t)stream);
    return ffn_bwd_t<float>(go, xd, h, a, offsets, kept_rows, E, max_rows, M, F, w1, w2, t, g_w1, g_b1, g_w2, g_b2, gx,
                            accumulate, gelu_bwd, (hipStream_t)stream);
}

extern "C" int mole_gemm_nt(const void *a, const void *b, int dtype, int rows, int N, int K, float *c,
                            mole_stream_t stream) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "mole_gemm_nt: bad dtype %d", dtype);
    MOLE_REQUIRE(rows >= 0 && N > 0 && K > 0 && K % (dtype == MOLE_BF16 ? 8 : 4) == 0, "mole_gemm_nt: bad sizes rows=%d N=%d K=%d", rows, N, K);
    if (rows == 0) return 0;
    MOLE_REQUIRE(a && b && c && al16(a) && al16(b), "mole_gemm_nt: null or misaligned pointer");
    GemmArgs g{};
    g.single_rows = rows; g.E = 1;
    g.A = a; g.lda = K; g.B = b; g.ldb = K; g.N = N; g.K = K; g.C = c; g.ldc = N;
    const int tiles = ceil_div(rows, TBM) * ceil_div(N, TBN);
    if (dtype == MOLE_BF16) return run_gemm<bf16_t, false, false, false, EPI_F32>(g, rows, tiles, (hipStream_t)stream, MOLE_K_GEMM_NT);
    return launch_gemm<float, false, false, false, TBM, TBN, EPI_F32>(g, tiles, (hipStream_t)stream, MOLE_K_GEMM_NT);
}

extern "C" int mole_gemm_nn(const void *a, const void *b, int dtype, int rows, int N, int K, void *c,
                            mole_stream_t stream) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "mole_gemm_nn: bad dtype %d", dtype);
    const int epc = dtype == MOLE_BF16 ? 8 : 4;
    MOLE_REQUIRE(rows >= 0 && N > 0 && K > 0 && K % epc == 0 && N % epc == 0, "mole_gemm_nn: bad sizes rows=%d N=%d K=%d", rows, N, K);
    if (rows == 0) return 0;
    MOLE_REQUIRE(a && b && c && al16(a) && al16(b) && al16(c), "mole_gemm_nn: null or misaligned pointer");
    GemmArgs g{};
    g.single_rows = rows; g.E = 1;
    g.A = a; g.lda = K; g.B = b; g.ldb = N; g.N = N; g.K = K; g.C = c; g.ldc = N;
    const int tiles = ceil_div(rows, TBM) * ceil_div(N, TBN);
    if (dtype == MOLE_BF16) return run_gemm<bf16_t, false, true, false, EPI_STORE>(g, rows, tiles, (hipStream_t)stream, MOLE_K_GEMM_NT);
    return launch_gemm<float, false, true, false, TBM, TBN, EPI_STORE>(g, tiles, (hipStream_t)stream, MOLE_K_GEMM_NT);
}

extern "C" int mole_gemm_tn(const void *a, const void *b, int dtype, int rows, int Mo, int N, void *c,
                            mole_stream_t stream) {
    MOLE_REQUIRE(dtype == MOLE_F32 || dtype == MOLE_BF16, "mole_gemm_tn: bad dtype %d", dtype);
    const int epc = dtype == MOLE_BF16 ? 8 : 4;
    MOLE_REQUIRE(rows >= 0 && N > 0 && Mo > 0 && Mo % epc == 0 && N % epc == 0, "mole_gemm_tn: bad sizes rows=%d Mo=%d N=%d", rows, Mo, N);
    MOLE_REQUIRE(c && al16(c) && (rows == 0 || (a && b && al16(a) && al16(b))), "mole_gemm_tn: null or misaligned pointer");
    GemmArgs g{};
    g.single_rows = rows; g.E = 1;      // one group whose contraction runs over all rows (zero rows: c = 0)
    g.A = a; g.lda = Mo; g.B = b; g.ldb = N; g.M = Mo; g.N = N; g.C = c; g.ldc = N; g.strideC = (long)Mo * N;
    const int tiles = ceil_div(Mo, TBM) * ceil_div(N, TBN);
    if (dtype == MOLE_BF16) return launch_gemm<bf16_t, true, true, true, TBM, TBN, EPI_WGRAD>(g, tiles, (hipStream_t)stream, MOLE_K_GEMM_NT);
    return launch_gemm<float, true, true, true, TBM, TBN, EPI_WGRAD>(g, tiles, (hipStream_t)stream, MOLE_K_GEMM_NT);
}
