// fp32 grouped GEMM for gfx950: the fast path of the six expert-FFN products in the reference's own dtype
// (MOLE/cpp/define.hpp:152-155 - fp32 is the only type its kernels are instantiated for; the products are
// _BatchRecord::bffn_fwd / bffn_bwd, MOLE/cpp/core.cpp:344-356, 381-414).
//
// v_mfma_f32_32x32x2_f32 keeps a SIMD's matrix pipe busy for 64 cycles and consumes one register of each operand,
// so the arithmetic leaves room for everything else - as long as something else is ready to issue.  The kernel is
// therefore built for several independent blocks per CU rather than one large one: a block of 4 waves (2 x 2) owns a
// BM x BN tile (64 x 128 for the row-ragged products, 128 x 128 for the weight gradients), its operand stages of 16
// of K come from HBM/L2 straight into a ring of three or four LDS stages (global_load_lds_dwordx4, one barrier per
// stage), and the fragments of stage s+1 are read into registers while the MFMAs of stage s run, the loads and reads
// dealt out between the MFMAs.  Two to four blocks share a CU.
//
// LDS images (the 16-byte piece a lane's load fills is fixed by the hardware; which global address it fetches
// is ours to choose, so any permutation of pieces is free):
//   * K-contiguous operand -> [row][4 x 16 B], piece index XORed with swz4(row); a ds_read_b128 gives a lane four
//     consecutive k of its row.  MFMA step (kk, j) therefore contracts k = 8 kk + j (lanes 0-31) and 8 kk + 4 + j
//     (lanes 32-63) - any pairing of k is as good as any other as long as both operands use the same.
//   * K-strided operand    -> [k][rows x 4 B] as it lies in HBM, the 16-byte piece index XORed with 8 on k-rows with
//     bit 2 set (the two k-rows one MFMA step reads then fall into different banks).  A wave's two 32-row blocks are
//     the even and the odd rows of its 64: one ds_read_b64 per step serves both.
// The m-side operand feeds the MFMA's first slot and the n-side the second, so the 32 lanes of a half wave hold 32
// consecutive (or, K-strided, 64 consecutive in pairs) columns of one result row: stores are whole 128- or 256-byte
// row segments straight from the accumulators.
#include "gemm.h"
#include "lds_dma.h"

namespace mole {
namespace {

constexpr int F_BK = 16;          // k per stage: 64 bytes of a K-contiguous row
constexpr int F_THREADS = 256;    // 4 waves, 2 x 2

template <int BM, int BN, int NSTAGE> struct FTile {
    static constexpr int TMW = BM / 64, TNW = BN / 64;        // 32-row blocks per wave on either side
    static constexpr int M_BYTES = BM * F_BK * 4, N_BYTES = BN * F_BK * 4, STAGE = M_BYTES + N_BYTES;
    static constexpr int LM = BM / 64, LN = BN / 64, L = LM + LN;   // 1-KiB loads per wave and stage
    static constexpr int LDS_BYTES = NSTAGE * STAGE;
};

// Per-lane byte offsets of the loads a wave issues for one stage of an operand tile, relative to the tile's first
// element at the stage's first k.  Wave w's load i fills LDS bytes [(4 i + w) 1024, +1024) of the tile.  Rows
// (k-rows) past the operand's end are clamped to the last valid one: what lands for them is finite data that only
// reaches results which are not stored - except along a ragged contraction, whose tail is zeroed in LDS.
template <int ROWS, bool KS> struct FOff {
    static constexpr int NL = ROWS / 64;
    uint32_t off[NL];
    __device__ __forceinline__ void init(long ld, int r_left, int k_left) {
        const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            if constexpr (!KS) {
                const int row = (4 * i + w) * 16 + (lane >> 2);
                const int c = (lane & 3) ^ swz4(row);
                off[i] = (uint32_t)(min(row, r_left - 1) * ld * 4 + c * 16);
            } else {
                constexpr int SPR = ROWS / 4, KPL = 64 / SPR;      // 16-byte pieces per k-row, k-rows per load
                const int kr = (4 * i + w) * KPL + lane / SPR;
                const int c = (lane % SPR) ^ (((kr >> 2) & 1) << 3);
                off[i] = (uint32_t)(min(kr, k_left - 1) * ld * 4 + min(c * 4, r_left - 4) * 4);
            }
        }
    }
};

// The fragments of one stage for the NB 32-row blocks of a wave on one side.  get(b, kk, j): the lane's operand
// register for block b in MFMA step (kk, j).
template <int ROWS, bool KS, int NB> struct FFrag {
    float v[8 * NB];
    __device__ __forceinline__ void read(const char *tile, uint32_t off0, uint32_t off1) {
        if constexpr (!KS) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int kk = 0; kk < 2; ++kk) {
                    const float4 t = *reinterpret_cast<const float4 *>(tile + (kk ? off1 : off0) + b * 2048);
                    v[(b * 2 + kk) * 4 + 0] = t.x; v[(b * 2 + kk) * 4 + 1] = t.y;
                    v[(b * 2 + kk) * 4 + 2] = t.z; v[(b * 2 + kk) * 4 + 3] = t.w;
                }
        } else {
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const char *p = tile + off0 + (8 * kk + j) * (ROWS * 4);
                    if constexpr (NB == 2) {
                        const float2 t = *reinterpret_cast<const float2 *>(p);
                        v[(kk * 4 + j) * 2] = t.x; v[(kk * 4 + j) * 2 + 1] = t.y;
                    } else {
                        v[kk * 4 + j] = *reinterpret_cast<const float *>(p);
                    }
                }
        }
    }
    __device__ __forceinline__ float get(int b, int kk, int j) const {
        if constexpr (!KS) return v[(b * 2 + kk) * 4 + j]; else return v[(kk * 4 + j) * NB + b];
    }
    // per-lane LDS byte offsets inside the operand tile; blk0: the wave's first 32-row block
    static __device__ __forceinline__ void offsets(int blk0, uint32_t &off0, uint32_t &off1) {
        const int lane = threadIdx.x & 63, lr = lane & 31, h = lane >> 5;
        if constexpr (!KS) {
            const int row = blk0 * 32 + lr;
            const int c0 = h ^ swz4(row);          // swz4 does not depend on the block (bits 1-3 of the row)
            off0 = (uint32_t)(row * 64 + c0 * 16);
            off1 = (uint32_t)(row * 64 + (c0 ^ 2) * 16);
        } else {
            const int lb = (blk0 * 32 + NB * lr) * 4;                     // logical byte inside the k-row
            off0 = (uint32_t)(4 * h * (ROWS * 4) + ((((lb >> 4) ^ (h << 3)) << 4) | (lb & 15)));
            off1 = 0;
        }
    }
};

template <int BM, int BN, int NSTAGE, int BPC, bool M_KS, bool N_KS, bool WG, int EPI>
__global__ __launch_bounds__(F_THREADS, BPC) void gemm_f32_kernel(const GemmArgs g) {
    typedef FTile<BM, BN, NSTAGE> TL;
    constexpr int F_NSTAGE = NSTAGE;
    constexpr int TMW = TL::TMW, TNW = TL::TNW, L = TL::L;
    extern __shared__ __align__(16) char smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // ---- which tile am I?  Blocks are dealt round-robin to the 8 XCDs (block b runs on XCD b mod 8): every XCD
    //      takes a contiguous range of the real tiles, so that neighbours share operands in its L2.  For row-ragged
    //      products the number of real tiles is only known here (the grid is sized for the worst case).
    const int n_tiles = (g.N + BN - 1) / BN;
    int e, mt, nt, m_ext, k_ext;
    long row0;
    if constexpr (!WG) {
        const bool single = g.offsets == nullptr;
        const int nE = single ? 1 : g.E;
        int part = 0;
        for (int ee = lane; ee < nE; ee += WAVE) part += ((single ? g.single_rows : g.kept[ee]) + BM - 1) / BM;
        for (int d = WAVE / 2; d >= 1; d >>= 1) part += __shfl_xor(part, d, WAVE);
        const int total = part * n_tiles;
        const int per_xcd = (total + 7) >> 3;
        const int slot = blockIdx.x >> 3;
        const int t = (blockIdx.x & 7) * per_xcd + slot;
        if (slot >= per_xcd || t >= total) return;
        const int mtg = t / n_tiles;
        nt = t % n_tiles;
        int run = 0, found = -1, fmt = 0;
        for (int base = 0; base < nE && found < 0; base += WAVE) {
            const int ee = base + lane;
            const int tiles = ee < nE ? ((single ? g.single_rows : g.kept[ee]) + BM - 1) / BM : 0;
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
        m_ext = single ? g.single_rows : g.kept[e];
        row0 = single ? 0 : g.offsets[e];
        k_ext = g.K;
    } else {
        const int t = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
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
    e = __builtin_amdgcn_readfirstlane(e);
    mt = __builtin_amdgcn_readfirstlane(mt);
    nt = __builtin_amdgcn_readfirstlane(nt);
    m_ext = __builtin_amdgcn_readfirstlane(m_ext);
    k_ext = __builtin_amdgcn_readfirstlane(k_ext);
    row0 = ((long)__builtin_amdgcn_readfirstlane((int)(row0 >> 32)) << 32) | (unsigned)__builtin_amdgcn_readfirstlane((int)row0);
    const int m0 = mt * BM, n0 = nt * BN;
    const float *Mp = (const float *)g.A + row0 * g.lda;
    const float *Np = WG ? (const float *)g.B + row0 * g.ldb : (const float *)g.B + (long)e * g.strideB;
    const int wm = wave >> 1, wn = wave & 1;

    f32x16 acc[TMW][TNW];
#pragma unroll
    for (int i = 0; i < TMW; ++i)
#pragma unroll
        for (int j = 0; j < TNW; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

    // Operand sums over the contraction (the bias gradients: sums of go and of t over an expert's rows, torch::sum_out
    // in MOLE/cpp/core.cpp:399, 408) ride along in the weight-gradient blocks that see the whole operand once: the
    // first n-tile of every m-tile for the m-side, the first m-tile of every n-tile for the n-side.  The wave row or
    // column that holds the operand's fragments adds them up as they pass, four partial sums per column.
    int sum_side = 0;
    if constexpr (WG) {
        if (g.colsum != nullptr) {
            if (g.colsum_side == 1 && nt == 0 && wn == 0) sum_side = 1;
            if (g.colsum_side == 2 && mt == 0 && wm == 0) sum_side = 2;
        }
    }
    constexpr int SB = TMW > TNW ? TMW : TNW;
    float psum[4][SB];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int b = 0; b < SB; ++b) psum[j][b] = 0.f;

    const int nk = (k_ext + F_BK - 1) / F_BK;
    if (nk > 0) {
        const int kl = k_ext - (nk - 1) * F_BK;     // k-rows of the last stage (a row-ragged product's K is whole stages)
        FOff<BM, M_KS> om, cm;
        FOff<BN, N_KS> on, cn;
        om.init(g.lda, m_ext - m0, F_BK);
        on.init(g.ldb, g.N - n0, F_BK);
        if constexpr (WG) { cm.init(g.lda, m_ext - m0, kl); cn.init(g.ldb, g.N - n0, kl); }
        const char *bm = uniform_ptr(M_KS ? Mp + m0 : Mp + (long)m0 * g.lda);
        const char *bn = uniform_ptr(N_KS ? Np + n0 : Np + (long)n0 * g.ldb);
        const long step_m = M_KS ? g.lda * (F_BK * 4) : F_BK * 4;
        const long step_n = N_KS ? g.ldb * (F_BK * 4) : F_BK * 4;
        const uint32_t lds_w = lds_offset_of(smem) + wave * 1024;
        // load j of stage s (the m-side tile's loads come first) into ring buffer s mod NSTAGE; stages are issued in
        // order, the bases advance after a stage's last load
        auto issue_one = [&](int s, int j) __attribute__((always_inline)) {
            const uint32_t dst = lds_w + (s % F_NSTAGE) * TL::STAGE;
            const bool last = WG && s == nk - 1;
            if (j < TL::LM) {
                uint32_t o = om.off[j];
                if constexpr (WG) o = last ? cm.off[j] : o;
                dma16s(bm, o, dst + j * 4096);
            } else {
                uint32_t o = on.off[j - TL::LM];
                if constexpr (WG) o = last ? cn.off[j - TL::LM] : o;
                dma16s(bn, o, dst + TL::M_BYTES + (j - TL::LM) * 4096);
            }
            if (j == L - 1) { bm += step_m; bn += step_n; }
        };
        auto issue = [&](int s) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < L; ++j) issue_one(s, j);
        };
        // ragged contraction: zero the k-rows past its end in the last stage (both tiles are [k][rows] there)
        auto zero_tail = [&](int buf) __attribute__((always_inline)) {
            char *b = smem + buf * TL::STAGE;
            for (int idx = threadIdx.x; idx < (F_BK - kl) * (BM / 4); idx += F_THREADS)
                *reinterpret_cast<float4 *>(b + kl * (BM * 4) + idx * 16) = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int idx = threadIdx.x; idx < (F_BK - kl) * (BN / 4); idx += F_THREADS)
                *reinterpret_cast<float4 *>(b + TL::M_BYTES + kl * (BN * 4) + idx * 16) = make_float4(0.f, 0.f, 0.f, 0.f);
            __syncthreads();
        };
        uint32_t fm0, fm1, fn0, fn1;
        FFrag<BM, M_KS, TMW>::offsets(wm * TMW, fm0, fm1);
        FFrag<BN, N_KS, TNW>::offsets(wn * TNW, fn0, fn1);
        FFrag<BM, M_KS, TMW> ma, mb;
        FFrag<BN, N_KS, TNW> na, nb;

#pragma unroll
        for (int s = 0; s < F_NSTAGE - 1; ++s)
            if (s < nk) issue(s);
        if (F_NSTAGE == 4 && nk >= 3) __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * L));
        else if (nk >= 2) __builtin_amdgcn_s_waitcnt(waitcnt_vm(L));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        __builtin_amdgcn_s_barrier();
        if (WG && nk == 1 && kl < F_BK) zero_tail(0);
        ma.read(smem, fm0, fm1);
        na.read(smem + TL::M_BYTES, fn0, fn1);

        // One stage: the MFMAs of stage S on the fragments MC / NC.  With NEXT, first the hand-over to stage S + 1: wait
        // until this wave's share of it has landed, barrier; then, dealt out between the MFMAs so that the matrix pipe
        // always has the next one waiting, the loads that refill the buffer stage S - 1 has left and the fragment reads
        // of stage S + 1 into MN / NN.  (A wave issues in order: eight loads and reads in a row right after the barrier
        // left the pipe idle for a tenth of a 64 x 128 tile's stage.)  NEXT is a compile-time choice: were the fragment
        // reads under a run-time condition, the compiler could not tell how many LDS reads are outstanding at the first
        // MFMA and would wait for all of them, the ones just issued included.
        // Order of a stage's MFMAs: two waves on a SIMD that each alternate between two accumulators run at 0.85 of the
        // MFMA rate on this chip (measured with operands held in registers: one, three or four accumulators in turn, or
        // one wave per SIMD, all reach the full rate), so a wave with two cells runs its eight steps on one cell, then
        // on the other; with four cells they take turns.
#define MOLE_F32_STAGE(S, MC, NC, MN, NN, NEXT)                                                             \
        {                                                                                                   \
            const int s_ = (S);                                                                             \
            bool refill_ = false;                                                                           \
            const int nb_ = (s_ + 1) % F_NSTAGE;                                                            \
            if constexpr (NEXT) {                                                                           \
                if (F_NSTAGE == 4 && s_ + 2 < nk) __builtin_amdgcn_s_waitcnt(waitcnt_vm(L));                \
                else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));                                             \
                __builtin_amdgcn_s_barrier();                                                               \
                refill_ = s_ + F_NSTAGE - 1 < nk;                                                           \
                if (WG && s_ + 1 == nk - 1 && kl < F_BK) zero_tail(nb_);                                    \
            }                                                                                               \
            constexpr int CELLS_ = TMW * TNW, NM_ = 8 * CELLS_, G_ = NM_ / 8;                               \
            _Pragma("unroll") for (int grp = 0; grp < 8; ++grp) {                                           \
                _Pragma("unroll") for (int u = 0; u < G_; ++u) {                                            \
                    const int n_ = grp * G_ + u;                                                            \
                    const int cell_ = CELLS_ == 2 ? n_ / 8 : n_ % CELLS_, step_ = CELLS_ == 2 ? n_ % 8 : n_ / CELLS_; \
                    const int tm = cell_ / TNW, tn = cell_ % TNW, kk = step_ / 4, j = step_ % 4;            \
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(MC.get(tm, kk, j), NC.get(tn, kk, j), acc[tm][tn], 0, 0, 0); \
                }                                                                                           \
                if constexpr (NEXT) {                                                                       \
                    if (grp < L && refill_) issue_one(s_ + F_NSTAGE - 1, grp);                              \
                    if (grp == 0) MN.read(smem + nb_ * TL::STAGE, fm0, fm1);                                \
                    if (grp == 1) NN.read(smem + nb_ * TL::STAGE + TL::M_BYTES, fn0, fn1);                  \
                }                                                                                           \
                __builtin_amdgcn_sched_barrier(0);                                                          \
            }                                                                                               \
            if constexpr (WG) {                                                                             \
                if (sum_side == 1) {                                                                        \
                    _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)                                        \
                    _Pragma("unroll") for (int j = 0; j < 4; ++j)                                           \
                    _Pragma("unroll") for (int b = 0; b < TMW; ++b) psum[j][b] += MC.get(b, kk, j);         \
                } else if (sum_side == 2) {                                                                 \
                    _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)                                        \
                    _Pragma("unroll") for (int j = 0; j < 4; ++j)                                           \
                    _Pragma("unroll") for (int b = 0; b < TNW; ++b) psum[j][b] += NC.get(b, kk, j);         \
                }                                                                                           \
            }                                                                                               \
        }
        int s = 0;
        for (; s + 2 < nk; s += 2) {
            MOLE_F32_STAGE(s, ma, na, mb, nb, true)
            MOLE_F32_STAGE(s + 1, mb, nb, ma, na, true)
        }
        if (nk - s == 2) {
            MOLE_F32_STAGE(s, ma, na, mb, nb, true)
            MOLE_F32_STAGE(s + 1, mb, nb, ma, na, false)
        } else {
            MOLE_F32_STAGE(s, ma, na, mb, nb, false)
        }
#undef MOLE_F32_STAGE
    }

    if constexpr (WG) {
        if (sum_side != 0) {
            // a lane's fragments cover k-rows 8 kk + 4 (lane / 32) + j: the two half waves hold the two halves of the sum
            const int nbk = sum_side == 1 ? TMW : TNW;
            const int first = sum_side == 1 ? m0 + wm * 32 * TMW : n0 + wn * 32 * TNW;
            const int ext = sum_side == 1 ? m_ext : g.N;
            float *out = (float *)g.colsum + (long)e * ext;
#pragma unroll
            for (int b = 0; b < SB; ++b) {
                float v = (psum[0][b] + psum[1][b]) + (psum[2][b] + psum[3][b]);
                v += __shfl_xor(v, 32, WAVE);
                const int c = first + nbk * (lane & 31) + b;
                if (b < nbk && lane < 32 && c < ext) {
                    if (g.accumulate) v += out[c];
                    out[c] = v;
                }
            }
        }
    }

    // ---- epilogue.  acc[tm][tn][q] = C[m, n] with i = 8 (q / 4) + 4 (lane / 32) + q % 4 the row inside the m-block and
    //      lane % 32 the column inside the n-block; a K-strided side interleaves the wave's blocks (row 2 i + tm).
    const int lr = lane & 31, h = lane >> 5;
    float *Cb = (float *)g.C;
    long crow0 = row0;
    if constexpr (WG) { crow0 = 0; Cb += (long)e * g.strideC; }
    constexpr bool PAIR = N_KS && TNW == 2;         // a lane holds two adjacent columns: 8-byte accesses
    int ncol[TNW];
    float bias[TNW];
#pragma unroll
    for (int tn = 0; tn < TNW; ++tn) {
        ncol[tn] = N_KS ? n0 + wn * 32 * TNW + TNW * lr + tn : n0 + (wn * TNW + tn) * 32 + lr;
        bias[tn] = 0.f;
        if constexpr (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU)
            if (ncol[tn] < g.N) bias[tn] = ((const float *)g.bias)[(long)e * g.N + ncol[tn]];
    }
    auto row_of = [&](int tm, int q) {
        const int i = 8 * (q >> 2) + 4 * h + (q & 3);
        return M_KS ? m0 + wm * 32 * TMW + TMW * i + tm : m0 + (wm * TMW + tm) * 32 + i;
    };
#pragma unroll
    for (int tm = 0; tm < TMW; ++tm) {
        // GELU', accumulation: the old values of this block's 16 rows are fetched first, unconditionally (rows and
        // columns past the end read a clamped address and are not used), so that they are in flight together
        float old[16][TNW];
        if constexpr (EPI == EPI_DGELU || EPI == EPI_WGRAD) {
            if (EPI == EPI_DGELU || g.accumulate) {
                const float *src = EPI == EPI_DGELU ? (const float *)g.H : Cb;
#pragma unroll
                for (int q = 0; q < 16; ++q) {
                    const long r = crow0 + min(row_of(tm, q), m_ext - 1);
                    if constexpr (PAIR) {
                        const float2 t = *reinterpret_cast<const float2 *>(src + r * g.ldc + min(ncol[0], g.N - 2));
                        old[q][0] = t.x; old[q][1] = t.y;
                    } else {
#pragma unroll
                        for (int tn = 0; tn < TNW; ++tn) old[q][tn] = src[r * g.ldc + min(ncol[tn], g.N - 1)];
                    }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int m = row_of(tm, q);
            if (m >= m_ext) continue;
            float v[TNW], v2[TNW];
#pragma unroll
            for (int tn = 0; tn < TNW; ++tn) {
                v[tn] = acc[tm][tn][q];
                v2[tn] = 0.f;
                if constexpr (EPI == EPI_BIAS) {
                    v[tn] += bias[tn];
                } else if constexpr (EPI == EPI_BIAS_GELU) {
                    v[tn] += bias[tn];
                    v2[tn] = gelu_erf(v[tn]);
                } else if constexpr (EPI == EPI_DGELU) {
                    const float hv = old[q][tn];
                    v[tn] *= g.gelu_bwd == MOLE_GELU_BWD_TANH ? d_gelu_tanh(hv) : d_gelu_exact(hv);
                } else if constexpr (EPI == EPI_WGRAD) {
                    if (g.accumulate) v[tn] += old[q][tn];
                }
            }
            float *dst = Cb + (crow0 + m) * g.ldc;
            // The weight gradients (which nothing reads before the optimizer) leave with non-temporal stores: -2 us on
            // 8 x 2048 x 512.  For h, a and t it measured neutral to worse: the launches that follow read them.
            constexpr bool STREAM = EPI == EPI_WGRAD;
            auto put = [&](float *p, float x) __attribute__((always_inline)) {
                if constexpr (STREAM) __builtin_nontemporal_store(x, p); else *p = x;
            };
            auto put2 = [&](float *p, float x, float y) __attribute__((always_inline)) {
                typedef float f32x2 __attribute__((ext_vector_type(2)));
                if constexpr (STREAM) __builtin_nontemporal_store(f32x2{x, y}, reinterpret_cast<f32x2 *>(p));
                else *reinterpret_cast<float2 *>(p) = make_float2(x, y);
            };
            if constexpr (PAIR) {
                if (ncol[0] < g.N) {
                    put2(dst + ncol[0], v[0], v[1]);
                    if constexpr (EPI == EPI_BIAS_GELU) put2((float *)g.C2 + (crow0 + m) * g.ldc + ncol[0], v2[0], v2[1]);
                }
            } else {
#pragma unroll
                for (int tn = 0; tn < TNW; ++tn) {
                    if (ncol[tn] >= g.N) continue;
                    put(dst + ncol[tn], v[tn]);
                    if constexpr (EPI == EPI_BIAS_GELU) put((float *)g.C2 + (crow0 + m) * g.ldc + ncol[tn], v2[tn]);
                }
            }
        }
    }
}

template <int BM, int BN, int NSTAGE, int BPC, bool M_KS, bool N_KS, bool WG, int EPI>
int launch_f32(GemmArgs g, int tiles, hipStream_t st, int kid) {
    if (tiles <= 0) return 0;
    g.n_blocks = tiles;
    const int grid = (tiles + 7) & ~7;
    auto kern = gemm_f32_kernel<BM, BN, NSTAGE, BPC, M_KS, N_KS, WG, EPI>;
    // the LDS request also caps the blocks a CU takes: with room for more than BPC, the dispatcher fills some CUs
    // and leaves others short, and the launch lasts as long as the fullest
    constexpr int lds_min = 160 * 1024 / (BPC + 1) + 1024;
    constexpr int lds = FTile<BM, BN, NSTAGE>::LDS_BYTES > lds_min ? FTile<BM, BN, NSTAGE>::LDS_BYTES : lds_min;
    static bool attr_done = false;
    if (!attr_done) {
        MOLE_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        attr_done = true;
    }
    timed_launch(kid, kern, dim3(grid), dim3(F_THREADS), lds, st, g);
    MOLE_LAUNCH_CHECK();
    return 0;
}

template <int BM, int BN, int NSTAGE, int BPC>
int dispatch_f32(const GemmArgs &g, bool b_ks, bool wg, int epi, int max_rows, hipStream_t st, int kid) {
    const int n_tiles = ceil_div(g.N, BN);
    if (wg) {
        const int tiles = g.E * ceil_div(g.M, BM) * n_tiles;
        if (epi == EPI_WGRAD) return launch_f32<BM, BN, NSTAGE, BPC, true, true, true, EPI_WGRAD>(g, tiles, st, kid);
        return -100;
    }
    const int rows_bound = g.offsets ? max_rows : g.single_rows;
    const int tiles = (rows_bound / BM + (g.offsets ? g.E : 1)) * n_tiles;     // every expert may end in a partial tile
    if (!b_ks) {
        if (epi == EPI_BIAS_GELU) return launch_f32<BM, BN, NSTAGE, BPC, false, false, false, EPI_BIAS_GELU>(g, tiles, st, kid);
        if (epi == EPI_DGELU) return launch_f32<BM, BN, NSTAGE, BPC, false, false, false, EPI_DGELU>(g, tiles, st, kid);
    } else {
        if (epi == EPI_BIAS) return launch_f32<BM, BN, NSTAGE, BPC, false, true, false, EPI_BIAS>(g, tiles, st, kid);
        if (epi == EPI_STORE) return launch_f32<BM, BN, NSTAGE, BPC, false, true, false, EPI_STORE>(g, tiles, st, kid);
    }
    return -100;
}

}  // namespace

// Tile shapes, from same-box sweeps on the reference's configuration (8 experts of about 1000 rows, M 512, F 2048) -
// durations in us of h = xd.w1^T + b1 | t = (go.w2^T) gelu'(h) | out = a.w2 + b2 | gx = t.w1 | the weight gradients:
//   128 x 128, 4 stages, 2 blocks per CU    153 | 150 |  -  |  -  | 126   (256 tiles of the two K = F products: one per CU)
//    64 x 128, 4 stages, 2 blocks per CU     -  |  -  | 127 | 124 | 131
//    64 x 128, 4 stages, 3 blocks per CU    155 | 145 |  -  |  -  | 131
//    64 x 128, 3 stages, 4 blocks per CU    144 | 145 |  -  |  -  | 127
//    64 x  64, 4 stages, 4 blocks per CU    154 | 163 | 128 | 127 |  -
//    64 x  64, 3 stages, 5 blocks per CU    152 | 159 |  -  |  -  |  -
//   128 x 128, 3 stages, 3 blocks per CU    176 | 171 |  -  |  -  | 125
// Row-ragged products take 64 x 128 tiles: with enough of them for four blocks per CU the shallower ring, otherwise
// two blocks per CU with the deeper one; weight gradients take 128 x 128.
// Whether the weight-gradient launch for g also produces the operand sums asked for in g.colsum.
bool gemm_f32_sums_operand(const GemmArgs &g) {
    return !(g.lda % 4 || g.ldb % 4 || g.ldc % 4 || g.N % 4 || g.N < 4 || g.M % 4 || g.M < 4);
}

int launch_gemm_f32(const GemmArgs &g, bool a_ks, bool b_ks, bool wg, int epi, int max_rows, hipStream_t st, int kid) {
    // what the direct-to-LDS path relies on: 16-byte rows, whole stages of K for row-ragged products
    if (g.lda % 4 || g.ldb % 4 || g.ldc % 4 || g.N % 4 || g.N < 4) return -100;
    if (!wg && (a_ks || g.K <= 0 || g.K % F_BK)) return -100;
    if (wg && (!a_ks || !b_ks || g.M % 4 || g.M < 4)) return -100;
    if (wg) return dispatch_f32<128, 128, 4, 2>(g, b_ks, wg, epi, max_rows, st, kid);
    const int rows = g.offsets ? max_rows : g.single_rows;
    const long tiles = (long)ceil_div(rows, 64) * ceil_div(g.N, 128);
    if (tiles >= 4 * 256) return dispatch_f32<64, 128, 3, 4>(g, b_ks, wg, epi, max_rows, st, kid);
    return dispatch_f32<64, 128, 4, 2>(g, b_ks, wg, epi, max_rows, st, kid);
}

}  // namespace mole
