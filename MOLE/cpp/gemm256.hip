// bf16 grouped GEMM for gfx950: the fast path of the six expert-FFN products.
//
// A block of 8 waves (2 wave rows x 4 wave columns, two waves per SIMD) owns a BM (m) x 256 (n) output tile, BM =
// 256 or up to 320; a wave covers BM/2 rows and 64 columns (BM/64 x 2 MFMA 32x32x16 blocks, fp32 accumulators).
// One block per CU.  (A build with -DMOLE_TUNING also carries the four-wave shapes and launch orders that were
// measured against this one and lost.)
// Operand tiles go from HBM/L2 straight into LDS (global_load_lds_dwordx4, no staging registers)
// through a ring of stages of 32 of K, several stages of loads in flight while one is consumed: with
// a single stage of look-ahead the loop ran at the memory latency, not at the MFMA rate.  One
// barrier per stage.  Each 16-byte piece is placed at a swizzled LDS position by choosing which
// global address the lane that owns the slot fetches:
//   * K-contiguous operand  -> LDS [row][4 x 16 B]; fragments read with ds_read_b128
//   * K-strided operand     -> LDS [k][rows x 2 B] as it lies in HBM; fragments read with
//                              ds_read_b64_tr_b16, the LDS transpose read
// The MFMA "A" slot is fed with the n-side operand and the "B" slot with the m-side operand, so the
// four consecutive accumulator rows a lane holds are four consecutive n; results leave through LDS
// as whole 128-byte rows.  A ragged m-tile runs only the 32-row blocks it has rows for.
#include "gemm.h"
#include "lds_dma.h"

#include <stdlib.h>

#include <type_traits>

namespace mole {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

constexpr int Q_BN = 256, Q_BK = 32;
constexpr int Q_N_OPERAND = Q_BN * Q_BK * 2;   // bytes of the n-side tile of one stage

// Geometry of a BM x 256 tile of TMB 32-row m-blocks computed by 4 WM waves: WM wave rows of TMB/WM m-blocks
// each, 4 wave columns of 64 columns each.  WM = 2 puts two waves on every SIMD: while one waits for
// the memory pipeline to accept a load or for a barrier, the other issues MFMAs.
template <int TMB, int WM> struct Tile {
    static constexpr int NW = 4 * WM, THREADS = 64 * NW, TMW = TMB / WM;
    static constexpr int BM = TMB * 32;
    static constexpr int M_ROWS = (BM + 16 * NW - 1) / (16 * NW) * (16 * NW);   // rows the waves' loads cover
    static constexpr int M_OPERAND = M_ROWS * Q_BK * 2;
    static constexpr int STAGE = M_OPERAND + Q_N_OPERAND;
    static constexpr int NSTAGE = TMB >= 8 ? 4 : 3;
    static constexpr int SLABS = NW * TMW * 32 * 128;                // the waves' epilogue staging areas
    static constexpr int LDS_BYTES = NSTAGE * STAGE > SLABS ? NSTAGE * STAGE : SLABS;
    static constexpr int BLOCKS_PER_CU = TMB >= 8 ? 1 : 2;
};

// One stage of the operand ring for a tile of which the first TMC 32-row blocks are live.  Of a K-contiguous
// m-side tile only the 64-row groups that hold live blocks are fetched and stored, so a light tile has
// smaller stages and its ring, in the same LDS, is deeper: light tiles do little arithmetic per stage and
// run at the memory latency divided by the stages in flight.
template <int TMB, int WM, bool M_KS, int TMC> struct Stage {
    typedef Tile<TMB, WM> TL;
    static constexpr int RPL = 16 * TL::NW;                                       // rows (or 16-byte slot groups) one load of every wave covers
    static_assert(!M_KS || TL::BM % RPL == 0, "a K-strided m-side tile must be whole load rounds wide");
    static constexpr int LM = M_KS ? TL::BM / RPL : (TMC * 32 + RPL - 1) / RPL;  // m-side loads per wave
    static constexpr int LN = Q_BN / RPL;
    static constexpr int L = LM + LN;                                             // loads per wave
    static constexpr int M_OPERAND = LM * RPL * Q_BK * 2;
    static constexpr int BYTES = M_OPERAND + Q_N_OPERAND;
    static constexpr int FIT = TL::NSTAGE * TL::STAGE / BYTES;
    static constexpr int NSTAGE = FIT > 6 ? 6 : FIT;
};

// ---- activation math for a bf16 result -----------------------------------------------------------
// On this chip every VALU instruction of an epilogue takes issue time from the MFMAs of the wave that
// shares its SIMD, and exp / rcp run at a quarter of the plain rate, so the three functions are evaluated
// as clamped odd polynomials: f(x) = v q(v^2), v = clamp(x / c, -1, 1), fitted (near-minimax, Lawson
// iteration) to erf(x / sqrt 2) and to the odd parts of the two GELU derivatives.  Beyond the clamp the
// functions are constant to within the stated error.  Absolute errors in fp32 Horner evaluation:
// erf 5.8e-5, derivatives 1.8e-4 - an order of magnitude below the bf16 rounding of the result.
// gelu(x) = x (1/2 + 1/2 erf(x / sqrt 2)).  The fit of erf(x / sqrt 2) is v q(v^2) in v = clamp(x / 4, -1, 1); with every
// coefficient scaled by a power of two (c_k / (8 * 16^k): exact in binary floating point, the Horner steps round as
// before) the same polynomial is evaluated in v = clamp(x, -4, 4) itself and delivers 1/2 erf directly:
// clamp, square, eight FMAs, one FMA for the 1/2 and the product with x - twelve instructions, no scaling of x, no
// separate x / 2.  Beyond the clamp erf is +-1 to within the fit's error, so x (1/2 +- 1/2) is x or 0 as it should be.
__device__ __forceinline__ float fast_gelu_erf(float x) {
    constexpr float c[9] = {3.19138169f / 8.0f,
                            -8.50055408f / (8.0f * 16.0f),
                            20.229044f / (8.0f * 256.0f),
                            -37.1561737f / (8.0f * 4096.0f),
                            51.8556824f / (8.0f * 65536.0f),
                            -52.8050575f / (8.0f * 1048576.0f),
                            36.4542885f / (8.0f * 16777216.0f),
                            -15.039053f / (8.0f * 268435456.0f),
                            2.77038407f / (8.0f * 4294967296.0f)};
    const float v = __builtin_amdgcn_fmed3f(x, -4.0f, 4.0f);
    const float t = v * v;
    float q = c[8];
#pragma unroll
    for (int k = 7; k >= 0; --k) q = fmaf(q, t, c[k]);
    return x * fmaf(v, q, 0.5f);
}
// The two GELU derivatives share the clamp (4.5) and the degree, so the variant is a choice of coefficients,
// made once per tile, not a branch per element: tanh form = what the reference's backward multiplies by
// (MOLE/cpp/gelu.cu:3-14), exact form = Phi(x) + x phi(x).  d(x) = 1/2 + v q(v^2), v = clamp(x / 4.5, -1, 1); as above
// the polynomial is evaluated in v = clamp(x, -4.5, 4.5) with the coefficients divided by 4.5^(2k+1) (in double
// precision, then rounded once: 4.5 is not a power of two).
struct DGeluCoef {
    float c[10];
    __device__ __forceinline__ void select(bool tanh_form) {
        constexpr double ct[10] = {3.58895016, -24.237009, 110.279869, -345.395355, 772.538513,
                                   -1226.4845, 1338.11902, -946.521179, 388.703674, -70.0920258};
        constexpr double ce[10] = {3.58931732, -24.1413288, 108.150215, -329.418243, 711.674683,
                                   -1091.27979, 1154.8053, -796.700195, 320.776367, -56.9563408};
        double s = 1.0 / 4.5;
#pragma unroll
        for (int i = 0; i < 10; ++i) {
            c[i] = (float)((tanh_form ? ct[i] : ce[i]) * s);
            s *= 1.0 / (4.5 * 4.5);
        }
    }
    __device__ __forceinline__ float operator()(float x) const {
        const float v = __builtin_amdgcn_fmed3f(x, -4.5f, 4.5f);
        const float t = v * v;
        float q = c[9];
#pragma unroll
        for (int k = 8; k >= 0; --k) q = fmaf(q, t, c[k]);
        return fmaf(v, q, 0.5f);
    }
};

// ---- operand tiles in LDS -------------------------------------------------------------------------
// A stage holds 32 of K.  Every lane always issues its load (no divergent branches in the K loop):
// rows past the operand's extent are clamped to the last valid row / 16-byte piece.  What lands in
// LDS for them is real, finite data that only contributes to output rows or columns the epilogue
// does not store - except along a ragged contraction length, which zero_k_tail() repairs.
//
// K-contiguous operand, element (r, k) at p[r*ld + k]: LDS [ROWS][4 x 16 B], the chunk index XORed
// with swz4(row), chosen so that the 16 rows a ds_read_b128 pass touches (and any 8 aligned rows)
// fall into distinct bank groups of the 64-bank LDS.
// With NW waves, wave w's load i fills LDS bytes [(NW i + w)*1024, +1024) = rows 16(NW i + w) .. +16.
// Per-lane byte offsets of the ROWS/(16 NW) loads a wave issues for one stage of an operand tile, relative to
// the tile's first element at the stage's first k (what the scalar base points at).  r_left = rows of the
// operand from the tile's first row on, k_left = k-rows from the stage's first k on (only the last stage
// of a ragged contraction has fewer than 32).
template <int ROWS, int NW> struct OffKC {
    uint32_t off[ROWS / (16 * NW)];
    __device__ __forceinline__ void init(long ld, int r_left) {
        const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
        for (int i = 0; i < ROWS / (16 * NW); ++i) {
            const int row = (NW * i + w) * 16 + (lane >> 2);
            const int c = (lane & 3) ^ swz4(row);
            off[i] = (uint32_t)(min(row, r_left - 1) * ld * 2 + c * 16);
        }
    }
};
// K-strided operand, element (r, k) at p[k*ld + r]: LDS [32 k][ROWS x 2 B] as it lies in HBM, the
// 32-byte granule index XORed with (k & 3) << 1 (conflict-free transpose reads, see frag_ks).
// A k-row has ROWS/8 slots of 16 bytes; a wave load of 1 KiB covers 512/ROWS k-rows.
template <int ROWS, int NW> struct OffKS {
    uint32_t off[ROWS / (16 * NW)];
    __device__ __forceinline__ void init(long ld, int r_left, int k_left) {
        constexpr int SPR = ROWS / 8;          // 16-byte slots per k-row
        constexpr int KPL = 64 / SPR;          // k-rows per wave load
        const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
        for (int i = 0; i < ROWS / (16 * NW); ++i) {
            const int kr = (NW * i + w) * KPL + lane / SPR;
            const int pc = lane % SPR;                                        // physical 16-byte slot in the k-row
            const int c = ((((pc >> 1) ^ ((kr & 3) << 1)) << 1) | (pc & 1));  // logical 16-byte chunk
            off[i] = (uint32_t)(min(kr, k_left - 1) * ld * 2 + min(c * 8, r_left - 8) * 2);
        }
    }
};
template <int ROWS, int NW, bool KS> struct Off;
template <int ROWS, int NW> struct Off<ROWS, NW, false> : OffKC<ROWS, NW> {};
template <int ROWS, int NW> struct Off<ROWS, NW, true> : OffKS<ROWS, NW> {};
// zero the k-rows [k_valid, 32) of a K-strided tile (the last, partial stage of a weight gradient)
template <int ROWS, int THREADS> __device__ __forceinline__ void zero_k_tail(char *lds, int k_valid) {
    for (int idx = threadIdx.x; idx < (Q_BK - k_valid) * (ROWS / 8); idx += THREADS)
        *reinterpret_cast<uint4 *>(lds + k_valid * (ROWS * 2) + idx * 16) = make_uint4(0, 0, 0, 0);
}

// ---- MFMA fragments: 8 bf16 of k for row (lane % 32) of 32-row block tb, k-sub-step kk (16 of k) --
__device__ __forceinline__ bf16x8 frag_kc(const char *lds, int tb, int kk) {
    const int lane = threadIdx.x & 63;
    const int row = tb * 32 + (lane & 31);
    const int chunk = (2 * kk + (lane >> 5)) ^ swz4(row);
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(lds + row * 64 + chunk * 16));
}
// ds_read_b64_tr_b16: in a group of 16 lanes, lane 4r+q supplies the address of 4 consecutive values
// of k-row r, and lane i receives column i of that 4 x 16 block.  Two reads give 8 of k.
template <int ROWS> __device__ __forceinline__ bf16x8 frag_ks(const char *lds, int tb, int kk) {
    const int lane = threadIdx.x & 63;
    const int gq = lane >> 4, l = lane & 15;
    const int k = 16 * kk + 8 * (gq >> 1) + (l >> 2);                   // + 4 for the second read
    const int gran = (tb * 2 + (gq & 1)) ^ ((l >> 2) << 1);            // (k & 3) == l >> 2
    const char *a0 = lds + k * (ROWS * 2) + gran * 32 + (l & 3) * 8;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(a0));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(a0 + 4 * ROWS * 2));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, v);
}
template <bool KS, int ROWS> __device__ __forceinline__ bf16x8 frag(const char *lds, int tb, int kk) {
    if constexpr (KS) return frag_ks<ROWS>(lds, tb, kk); else return frag_kc(lds, tb, kk);
}

// first index of part P when N items are dealt to NP consecutive parts
template <int P, int NP, int N> constexpr int part_lo() { return P * N / NP; }

// The fragments one wave needs for a k-sub-step: its TMCW m-blocks (blocks wm*TMCW .. of the tile, of which
// the tile's first TMC are fetched) and its two 32-column n-blocks.
template <int TMB, int WM, bool M_KS, bool N_KS, int TMC, int TMCW> struct Frags {
    typedef Tile<TMB, WM> TL;
    static constexpr int NR = TMCW ? TMCW + 2 : 0;
    bf16x8 m[TMCW ? TMCW : 1], n[2];
    // the fragment reads of a k-sub-step, n-side first, dealt to NP parts
    template <int P, int NP> __device__ __forceinline__ void read_part(const char *stage, int wm, int wn, int kk) {
#pragma unroll
        for (int r = part_lo<P, NP, NR>(); r < part_lo<P + 1, NP, NR>(); ++r) {
            if (r < 2) n[r] = frag<N_KS, Q_BN>(stage + Stage<TMB, WM, M_KS, TMC>::M_OPERAND, wn * 2 + r, kk);
            else m[r - 2] = frag<M_KS, TL::BM>(stage, wm * TMCW + r - 2, kk);
        }
    }
    __device__ __forceinline__ void read(const char *stage, int wm, int wn, int kk) { read_part<0, 1>(stage, wm, wn, kk); }
    // the 2 TMCW MFMAs of a k-sub-step dealt to NP parts.  SUM: the last part adds one MFMA against a block of
    // ones, which sums one operand block over k: of the m-side (SUM 1; wave column i takes the wave row's
    // m-block i) or of the n-side (SUM 2; wave row j takes the wave column's n-block j).
    template <int P, int NP, int SUM> __device__ __forceinline__ void mma_part(f32x16 (&acc)[TL::TMW][2], f32x16 &sums, int wm, int wn) const {
#pragma unroll
        for (int i = part_lo<P, NP, 2 * TMCW>(); i < part_lo<P + 1, NP, 2 * TMCW>(); ++i)
            acc[i >> 1][i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(n[i & 1], m[i >> 1], acc[i >> 1][i & 1], 0, 0, 0);
        if constexpr (SUM != 0 && P == NP - 1) {
            const bf16_t one = (bf16_t)1.0f;
            const bf16x8 ones = {one, one, one, one, one, one, one, one};
            if constexpr (SUM == 1) {
#pragma unroll
                for (int i = 0; i < TMCW; ++i)
                    if (wn == i) sums = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, m[i], sums, 0, 0, 0);
            } else {
                if (wm == 0) sums = __builtin_amdgcn_mfma_f32_32x32x16_bf16(n[0], ones, sums, 0, 0, 0);
                else sums = __builtin_amdgcn_mfma_f32_32x32x16_bf16(n[1], ones, sums, 0, 0, 0);
            }
        }
    }
};

// Issues the asynchronous loads of the operand stages of one tile.  The two operand tiles are addressed
// by a scalar base (advanced by one stage of K after a stage's last load) plus per-lane offsets that stay
// fixed for the whole K loop.  Stages are fetched in order; past the last one the last is fetched again,
// harmlessly: it keeps the number of loads per stage, which the vmcnt arithmetic of the loop relies on.
// Of a K-contiguous m-side tile only the 64-row groups that hold live 32-row blocks (the first TMC) are fetched.
template <int TMB, int WM, bool M_KS, bool N_KS, bool WG, int TMC> struct Feeder {
    typedef Tile<TMB, WM> TL;
    typedef Stage<TMB, WM, M_KS, TMC> SG;
    static constexpr int LM = SG::LM, L = SG::L;
    Off<TL::M_ROWS, TL::NW, M_KS> om, cm;
    Off<Q_BN, TL::NW, N_KS> on, cn;
    const char *bm, *bn;
    long step_m, step_n;
    uint32_t lds_w;      // LDS address of ring buffer 0 + this wave's 1 KiB lane
    int nk;
    bool ragged_k;
    __device__ __forceinline__ void init(const bf16_t *Mp, long ldm, int m0, int m_ext, const bf16_t *Np, long ldn, int n0,
                                         int n_ext, int k_ext, char *smem, int wave) {
        if constexpr (M_KS) om.init(ldm, m_ext - m0, Q_BK); else om.init(ldm, m_ext - m0);
        if constexpr (N_KS) on.init(ldn, n_ext - n0, Q_BK); else on.init(ldn, n_ext - n0);
        ragged_k = WG && (k_ext & (Q_BK - 1));
        if constexpr (WG) {   // last stage of a ragged contraction: k-rows past the end are clamped to the last one
            cm.init(ldm, m_ext - m0, ragged_k ? (k_ext & (Q_BK - 1)) : Q_BK);
            cn.init(ldn, n_ext - n0, ragged_k ? (k_ext & (Q_BK - 1)) : Q_BK);
        }
        bm = uniform_ptr(M_KS ? Mp + m0 : Mp + (long)m0 * ldm);
        bn = uniform_ptr(N_KS ? Np + n0 : Np + (long)n0 * ldn);
        step_m = M_KS ? ldm * (Q_BK * 2) : Q_BK * 2;
        step_n = N_KS ? ldn * (Q_BK * 2) : Q_BK * 2;
        lds_w = lds_offset_of(smem) + __builtin_amdgcn_readfirstlane(wave * 1024);
        nk = (k_ext + Q_BK - 1) / Q_BK;
    }
    // loads [J0, J1) of stage s (the m-side tile's loads come first) into ring buffer buf
    template <int J0, int J1> __device__ __forceinline__ void issue(int s, int buf) {
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_w + buf * SG::BYTES);
        const bool clamp_k = WG && ragged_k && s >= nk - 1;
#pragma unroll
        for (int j = J0; j < J1; ++j) {
            if (j < LM) {
                uint32_t o = om.off[j];
                if constexpr (WG) o = clamp_k ? cm.off[j] : o;
                dma16s(bm, o, dst + j * (TL::NW * 1024));
            } else {
                uint32_t o = on.off[j - LM];
                if constexpr (WG) o = clamp_k ? cn.off[j - LM] : o;
                dma16s(bn, o, dst + SG::M_OPERAND + (j - LM) * (TL::NW * 1024));
            }
        }
        if (J1 == L && s + 1 < nk) { bm += step_m; bn += step_n; }
    }
};

__device__ __forceinline__ uint2 pack4(float a, float b, float c, float d) {
    const bf16x4 v = {(bf16_t)a, (bf16_t)b, (bf16_t)c, (bf16_t)d};
    return __builtin_bit_cast(uint2, v);
}
__device__ __forceinline__ void unpack4(uint2 u, float *f) {
    f[0] = __uint_as_float(u.x << 16);
    f[1] = __uint_as_float(u.x & 0xffff0000u);
    f[2] = __uint_as_float(u.y << 16);
    f[3] = __uint_as_float(u.y & 0xffff0000u);
}

// Waits until at most `behind` whole stages of L loads each (behind <= B; below 0 counts as 0), and X more loads if
// `extra`, are in flight (the instruction takes its count as an immediate, hence the chain).
template <int B, int L, int X> __device__ __forceinline__ void wait_stages_behind(int behind, bool extra) {
    if constexpr (B <= 0) {
        if (extra) __builtin_amdgcn_s_waitcnt(waitcnt_vm(X));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    } else {
        if (behind >= B) {
            if (extra) __builtin_amdgcn_s_waitcnt(waitcnt_vm(B * L + X));
            else __builtin_amdgcn_s_waitcnt(waitcnt_vm(B * L));
        } else {
            wait_stages_behind<B - 1, L, X>(behind, extra);
        }
    }
}

// The K loop.  Stage s (32 of K) lives in ring buffer s mod NSTAGE and is fetched NSTAGE-1 stages ahead.
// A wave cannot issue MFMAs while one of its loads waits for the memory pipeline to take it, so the loads
// of a stage are not issued in one burst: each half of an iteration is cut into parts, and a part issues
// its share of the loads, then its share of the fragment reads for the next sub-step, then its MFMAs.
// The second half of iteration s issues the first half of the loads of stage s+AHEAD, the first half of
// iteration s+1 the rest, into the buffer that stage s-1 has left.  One synchronisation point per
// iteration, between the halves: wait until this wave's share of stage s+1 has landed (newer stages may
// still be in flight), then the barrier.
// PART (measurement only, results are then meaningless): 1 leaves out the operand loads, 2 the fragment reads of the
// loop (the first stage's fragments are used throughout), 3 the barriers, 4 all three.
// BIAS: the accumulators start from the bias of their columns instead of zero (bias_raw: the 8 x 4 columns a lane
// holds, fetched before the operand loads and therefore landed when the first stage has), so that the epilogue adds
// nothing.
template <int TMB, int WM, bool M_KS, bool N_KS, bool WG, int TMC, int TMCW, int SUM, int PART = 0, bool BIAS = false>
__device__ __forceinline__ void main_loop(const bf16_t *Mp, long ldm, int m0, int m_ext, const bf16_t *Np, long ldn,
                                          int n0, int n_ext, int k_ext, char *smem, int wave, int wm, int wn,
                                          f32x16 (&acc)[Tile<TMB, WM>::TMW][2], f32x16 &sums, const uint2 (&bias_raw)[8]) {
    typedef Tile<TMB, WM> TL;
    typedef Stage<TMB, WM, M_KS, TMC> SG;
    constexpr int AHEAD = SG::NSTAGE - 1, NP = 4;
    typedef Feeder<TMB, WM, M_KS, N_KS, WG, TMC> FD;
    constexpr int L = FD::L, LH = L / 2;      // loads per wave per stage; the halves are LH and L - LH
    const int nk = __builtin_amdgcn_readfirstlane((k_ext + Q_BK - 1) / Q_BK);
    if (nk == 0) return;
    FD fd;
    fd.init(Mp, ldm, m0, m_ext, Np, ldn, n0, n_ext, k_ext, smem, wave);
    auto fix_tail = [&](int s, int buf) __attribute__((always_inline)) {   // ragged contraction: zero what lies past it in the last stage
        if (WG && s == nk - 1 && (k_ext & (Q_BK - 1))) {
            char *b = smem + buf * SG::BYTES;
            zero_k_tail<TL::BM, TL::THREADS>(b, k_ext & (Q_BK - 1));
            zero_k_tail<Q_BN, TL::THREADS>(b + SG::M_OPERAND, k_ext & (Q_BK - 1));
            __syncthreads();
        }
    };
    // SPLIT: with three or more stages in flight a stage's loads are spread over two halves (one iteration
    // of look-ahead is lost for the later half); with two, all of them go into the half after the barrier.
    constexpr bool SPLIT = AHEAD >= 3;
    constexpr bool NO_LOADS = PART == 1 || PART == 4, NO_READS = PART == 2 || PART == 4, NO_BARRIERS = PART == 3 || PART == 4;
    // Only stages that exist are fetched (but for one part of a stage, see below): the prologue stops at the
    // contraction's last stage, the last iterations issue nothing, and the waits count what is really in flight.
    // Fetching AHEAD stages past the end, as a loop with one kind of iteration does, costs a tile of K = 1024 a tenth
    // more loads, a one-stage tile of a nearly empty expert four times its loads, and the epilogue a wait for loads
    // that nothing reads.  The iterations without loads are a second copy of the loop body, compiled without them: the
    // same body with the loads under a (wave-uniform) condition ran 3-10 % slower, and a third copy for the one
    // iteration in between made the register allocator spill.
    constexpr int LX = SPLIT ? LH : L;        // loads of stage AHEAD - 1 that the prologue issues
    if constexpr (!NO_LOADS) {
#pragma unroll
        for (int s = 0; s < AHEAD - 1; ++s)
            if (s < nk) fd.template issue<0, L>(s, s);
        if (AHEAD - 1 < nk) fd.template issue<0, LX>(AHEAD - 1, AHEAD - 1);
    }
    // stage 0 has landed when no more is in flight than what was issued after it
    if (nk >= AHEAD) __builtin_amdgcn_s_waitcnt(waitcnt_vm((AHEAD - 2) * L + LX));
    else wait_stages_behind<AHEAD - 2, L, 0>(nk - 1, false);
    __builtin_amdgcn_s_barrier();
    if constexpr (BIAS) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            float b4[4];
            unpack4(bias_raw[c], b4);
#pragma unroll
            for (int tm = 0; tm < TMCW; ++tm)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[tm][c >> 2][4 * (c & 3) + j] = b4[j];
        }
    }
    fix_tail(0, 0);
    Frags<TMB, WM, M_KS, N_KS, TMC, TMCW> f0, f1;
    f0.read(smem, wm, wn, 0);
    if constexpr (NO_READS) f1.read(smem, wm, wn, 1);
    int cur_b = 0;                    // ring buffer of stage s
#define MOLE_HALF(ISSUE, P, J0, N, S_LOAD, BUF, FR, STAGE_PTR, KK, FM)                                    \
        if constexpr (!NO_LOADS && (ISSUE)) fd.template issue<(J0) + part_lo<P, NP, (N)>(), (J0) + part_lo<P + 1, NP, (N)>()>(S_LOAD, BUF); \
        if constexpr (!NO_READS) FR.template read_part<P, NP>(STAGE_PTR, wm, wn, KK);                       \
        FM.template mma_part<P, NP, SUM>(acc, sums, wm, wn);                                              \
        __builtin_amdgcn_sched_barrier(0);
    // One iteration (stage s).  ISSUE: the first half issues the rest of stage s + AHEAD - 1, the second the first
    // loads of stage s + AHEAD; WAIT: the wait for stage s + 1.
#define MOLE_ITER(ISSUE, WAIT)                                                                            \
    {                                                                                                     \
        const int nxt_b = cur_b + 1 == SG::NSTAGE ? 0 : cur_b + 1;                                        \
        const int free_b = cur_b == 0 ? SG::NSTAGE - 1 : cur_b - 1;     /* held stage s-1, takes stage s+AHEAD */ \
        const int fill_b = free_b == 0 ? SG::NSTAGE - 1 : free_b - 1;   /* takes the rest of stage s+AHEAD-1 */   \
        const char *cur = smem + cur_b * SG::BYTES;                                                       \
        const char *nxt = smem + nxt_b * SG::BYTES;                                                       \
        MOLE_HALF(ISSUE, 0, SPLIT ? LH : 0, SPLIT ? L - LH : 0, s + AHEAD - 1, fill_b, f1, cur, 1, f0)    \
        MOLE_HALF(ISSUE, 1, SPLIT ? LH : 0, SPLIT ? L - LH : 0, s + AHEAD - 1, fill_b, f1, cur, 1, f0)    \
        MOLE_HALF(ISSUE, 2, SPLIT ? LH : 0, SPLIT ? L - LH : 0, s + AHEAD - 1, fill_b, f1, cur, 1, f0)    \
        MOLE_HALF(ISSUE, 3, SPLIT ? LH : 0, SPLIT ? L - LH : 0, s + AHEAD - 1, fill_b, f1, cur, 1, f0)    \
        WAIT;                                                                                             \
        if constexpr (!NO_BARRIERS) __builtin_amdgcn_s_barrier();                                         \
        __builtin_amdgcn_sched_barrier(0);                                                                \
        fix_tail(s + 1, nxt_b);                                                                           \
        MOLE_HALF(ISSUE, 0, 0, SPLIT ? LH : L, s + AHEAD, free_b, f0, nxt, 0, f1)                         \
        MOLE_HALF(ISSUE, 1, 0, SPLIT ? LH : L, s + AHEAD, free_b, f0, nxt, 0, f1)                         \
        MOLE_HALF(ISSUE, 2, 0, SPLIT ? LH : L, s + AHEAD, free_b, f0, nxt, 0, f1)                         \
        MOLE_HALF(ISSUE, 3, 0, SPLIT ? LH : L, s + AHEAD, free_b, f0, nxt, 0, f1)                         \
        cur_b = nxt_b;                                                                                    \
    }
    int s = 0;
    // while stage s + AHEAD - 1 exists: its rest is issued, then the first loads of stage s + AHEAD (in the last of
    // these iterations that stage does not exist: LX loads that nothing reads, the only ones of a tile)
    for (; s + AHEAD - 1 < nk; ++s) MOLE_ITER(true, __builtin_amdgcn_s_waitcnt(waitcnt_vm((AHEAD - 2) * L)))
    // the last AHEAD - 1 iterations issue nothing; in flight behind stage s + 1: the stages after it and those LX loads
    const bool extra = nk >= AHEAD;
    for (; s < nk; ++s) MOLE_ITER(false, (wait_stages_behind<AHEAD - 2, L, LX>(nk - 2 - s, extra)))
#undef MOLE_ITER
#undef MOLE_HALF
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));   // nothing may still be writing LDS when the block retires
}

// The bias of the 8 x 4 columns a lane holds results for, as raw bf16 quadruples; fetched before the K loop
// so that the epilogue does not wait for it (zero bits are 0.0 in bf16).
template <int EPI> __device__ __forceinline__ void load_bias(const GemmArgs &g, int e, int n0, int lane, int wn, uint2 (&bias_raw)[8]) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        bias_raw[c] = make_uint2(0, 0);
        if constexpr (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU) {
            const int n = n0 + wn * 64 + (c >> 2) * 32 + 8 * (c & 3) + 4 * (lane >> 5);
            if (n < g.N) bias_raw[c] = *reinterpret_cast<const uint2 *>((const bf16_t *)g.bias + (long)e * g.N + n);
        }
    }
}

// The epilogue of one wave, whose first TMCW 32-row blocks hold live rows.  acc[tm][tn][4q+j] = C[m, n] with
// m = m0 + 32 tm + lane%32 (m0: the wave's first row) and n = n0 + 64 wn + 32 tn + 8 q + 4 (lane/32) + j.  A wave
// owns a (32 TMW) x 64 slab of the tile.  bf16 results go through the wave's own slab of LDS (the K loop is
// done with it) so that global memory sees whole 128-byte rows: 8 bytes per lane into LDS, then 16 bytes
// per lane out, 8 rows per store instruction.  The pre-activation that GELU' needs comes in the same way,
// in the opposite direction.  TMCW is a compile-time bound so that the work of different cells can be
// interleaved.  live: the wave's live rows.
template <int TMB, int WM, bool WG, int EPI, int TMC>
__device__ __forceinline__ void epilogue(const GemmArgs &g, f32x16 (&acc)[Tile<TMB, WM>::TMW][2], char *smem, int lane, int wave,
                                         int wn, int e, long row0, int m0, int n0, int m_ext, int live,
                                         const uint2 (&bias_raw)[8]) {
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
    if constexpr (TMC == 0) return;
    const int lm = lane & 31, h = lane >> 5;
    bf16_t *Cb = (bf16_t *)g.C;
    long crow0 = row0;
    if constexpr (WG) { crow0 = 0; Cb += (long)e * g.strideC; }
    const int nw0 = n0 + wn * 64;                   // first column of this wave's slab
    char *slab = smem + wave * (Tile<TMB, WM>::TMW * 32 * 128);
    const int jr = lane >> 3, jc = lane & 7;        // row-in-group / 16-byte column of the wide accesses
    const bool col_ok = nw0 + jc * 8 < g.N;

    // 8-byte cell (row, chunk, half): chunk ^ (row >> 1) & 7 and half ^ (row >> 4) & 1 make the 32 rows
    // one ds_write_b64 pass touches land in 32 distinct 8-byte bank groups
    auto slab_at = [&](int row, int chunk, int half) -> char * {
        return slab + row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4) + ((half ^ (row >> 4)) & 1) * 8;
    };
    // (a 16-byte access sees the two halves of a chunk swapped on rows with bit 4 set)
    // slab -> global: rows [0, live) of the slab, 128 bytes each
    // The large results - h, a, t and the weight gradients, 134-270 MB a launch, which no block of the same
    // launch reads - leave with non-temporal stores: ordinary stores let them push the operand panels of the
    // running K loops out of the L2 and the last-level cache.  Measured at 16 experts of 1024 x 4096 over 16384
    // rows (same-box A/B): h and a of the first product -11 us, the weight gradients -6 us and the GELU' product
    // that follows them -6 us, t of the GELU' product -4 us; the launches that read them later are MFMA-bound
    // and take them from HBM at no loss.  The small results (out, gx: 34 MB) stay ordinary: the row permutes
    // that read them next are memory-bound and lost more than the products gained.
    constexpr bool STREAM_OUT = EPI == EPI_BIAS_GELU || EPI == EPI_DGELU || EPI == EPI_WGRAD;
    // Addresses of the wide accesses: a wave-uniform 64-bit base (the slab's first row in the result, advanced by
    // scalar adds from row group to row group) plus a 32-bit per-lane byte offset that is computed once, so a store
    // costs no address arithmetic on the vector ALU; and the LDS reads of a batch of eight row groups are issued
    // before the first store, so that one LDS latency is waited for per batch instead of one per store.  (Written
    // row by row with the row test around the read and the store, each store waited for its own LDS read and
    // recomputed a 64-bit row * pitch product: two thirds of the epilogue's time apart from the activation.)
    const uint32_t pitch = (uint32_t)g.ldc * 2;                          // bytes between rows of the result
    const uint32_t lane_off = (uint32_t)jr * pitch + (uint32_t)jc * 16;  // this lane's 16 bytes of row jr
    // every row group and every column is stored (the same in all lanes)
    const bool full = __builtin_amdgcn_readfirstlane(live >= TMC * 32 && nw0 + 64 <= g.N) != 0;
    // LDS address of this lane's 16 bytes of row group `it` (rows 8 it + jr): with row = 8 it + jr the swizzle term
    // (row >> 1) & 7 is (jr >> 1) | ((it & 1) << 2), so two per-lane bases and a constant per row group suffice
    char *const wide0 = slab + jr * 128 + ((jc ^ (jr >> 1)) << 4);
    char *const wide1 = slab + jr * 128 + ((jc ^ (jr >> 1) ^ 4) << 4);
    auto wide_cell = [&](int it) -> char * { return ((it & 1) ? wide1 : wide0) + it * 1024; };
    auto fix_it = [&](uint4 v, int it) -> uint4 {      // rows with bit 4 set (it & 2) hold their halves swapped
        return (it & 2) ? make_uint4(v.z, v.w, v.x, v.y) : v;
    };
    typedef __attribute__((address_space(1))) char gchar;
    auto flush = [&](bf16_t *dst) __attribute__((always_inline)) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        gchar *gbase = (gchar *)((char *)dst + ((crow0 + m0) * g.ldc + nw0) * 2);
#pragma unroll
        for (int it0 = 0; it0 < TMC * 4; it0 += 8) {
            uint4 v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (it0 + i < TMC * 4) v[i] = fix_it(*reinterpret_cast<const uint4 *>(wide_cell(it0 + i)), it0 + i);
            auto put = [&](int i) __attribute__((always_inline)) {
                gchar *p = gbase + (size_t)(it0 + i) * 8 * pitch + lane_off;
                typedef __attribute__((address_space(1))) u32x4 g_u32x4;
                if constexpr (STREAM_OUT) __builtin_nontemporal_store(u32x4{v[i].x, v[i].y, v[i].z, v[i].w}, reinterpret_cast<g_u32x4 *>(p));
                else *reinterpret_cast<g_u32x4 *>(p) = u32x4{v[i].x, v[i].y, v[i].z, v[i].w};
            };
            if (full) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (it0 + i < TMC * 4) put(i);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (it0 + i < TMC * 4 && (it0 + i) * 8 + jr < live && col_ok) put(i);
            }
        }
    };
    // global -> slab, eight rows' loads in flight at a time.  Every load is issued, from an address clamped
    // into the operand (rows past the end read its last row, columns past the end its first column): what lands
    // in cells outside the live part is never written back, and a load under a condition would make the
    // compiler wait for all loads in flight at each one, so the eight would run one after the other.
    auto fill = [&](const bf16_t *src) __attribute__((always_inline)) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        // rows are counted from the slab's first row, or from the operand's last row when the slab starts past it
        const long first = min(crow0 + m0, crow0 + m_ext - 1);
        // byte offset of the last valid row, as far as the slab reaches (the row count is bounded before it meets the
        // pitch: an expert of 10^5 rows times a pitch of tens of KB does not fit 32 bits)
        const uint32_t last_off = (uint32_t)min(crow0 + m_ext - 1 - first, (long)(TMC * 32 - 1)) * pitch;
        const gchar *gbase = (const gchar *)((const char *)src + first * g.ldc * 2);
        const uint32_t col_off = col_ok ? (uint32_t)(nw0 + jc * 8) * 2 : 0u;
        const uint32_t row_off = (uint32_t)jr * pitch;
#pragma unroll
        for (int it0 = 0; it0 < TMC * 4; it0 += 8) {
            uint4 v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (it0 + i >= TMC * 4) continue;
                const uint32_t ro = min(row_off + (uint32_t)(it0 + i) * 8 * pitch, last_off);
                // read once, here: a non-temporal load keeps it from displacing the K loop's operands (-4 us)
                typedef __attribute__((address_space(1))) u32x4 g_u32x4;
                const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const g_u32x4 *>(gbase + ro + col_off));
                v[i] = make_uint4(w[0], w[1], w[2], w[3]);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (it0 + i < TMC * 4) *reinterpret_cast<uint4 *>(wide_cell(it0 + i)) = fix_it(v[i], it0 + i);
        }
    };

    if constexpr (EPI >= EPI_NONE) {
        // the K loop alone (mole_probe_kloop): results leave only under a condition that never holds, which is
        // enough to keep the accumulation alive
        if (g.K < 0) {
            float s = 0.f;
#pragma unroll
            for (int tm = 0; tm < TMC; ++tm)
#pragma unroll
                for (int tn = 0; tn < 2; ++tn)
#pragma unroll
                    for (int q = 0; q < 16; ++q) s += acc[tm][tn][q];
            ((float *)g.C)[threadIdx.x] = s;
        }
        return;
    }
    if constexpr (EPI == EPI_F32) {
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nw0 + tn * 32 + 8 * q + 4 * h;
                if (n >= g.N) continue;
#pragma unroll
                for (int tm = 0; tm < TMC; ++tm) {
                    const int m = m0 + tm * 32 + lm;
                    if (m >= m_ext) continue;
                    *reinterpret_cast<float4 *>((float *)g.C + (crow0 + m) * g.ldc + n) =
                        make_float4(acc[tm][tn][4 * q], acc[tm][tn][4 * q + 1], acc[tm][tn][4 * q + 2], acc[tm][tn][4 * q + 3]);
                }
            }
        return;
    }
    if constexpr (EPI == EPI_DGELU) fill((const bf16_t *)g.H);
    if constexpr (EPI == EPI_WGRAD) { if (g.accumulate) fill(Cb); }

    DGeluCoef dgelu;
    if constexpr (EPI == EPI_DGELU) dgelu.select(g.gelu_bwd == MOLE_GELU_BWD_TANH);
    // pass 0 writes C; for EPI_BIAS_GELU pass 1 writes C2 = gelu(h)
    constexpr int PASSES = EPI == EPI_BIAS_GELU ? 2 : 1;
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
#pragma unroll
        for (int tn = 0; tn < 2; ++tn) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nw0 + tn * 32 + 8 * q + 4 * h;
                (void)n;          // (the bias is in the accumulators already: the K loop started from it)
#pragma unroll
                for (int tm = 0; tm < TMC; ++tm) {
                    char *cell = slab_at(tm * 32 + lm, tn * 4 + q, h);
                    float v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = acc[tm][tn][4 * q + j];
                    if constexpr (EPI == EPI_BIAS_GELU) {
                        if (pass == 1) {
#pragma unroll
                            for (int j = 0; j < 4; ++j) v[j] = fast_gelu_erf(v[j]);
                        }
                    } else if constexpr (EPI == EPI_DGELU) {
                        float hv[4];
                        unpack4(*reinterpret_cast<const uint2 *>(cell), hv);
#pragma unroll
                        for (int j = 0; j < 4; ++j) v[j] *= dgelu(hv[j]);
                    } else if constexpr (EPI == EPI_WGRAD) {
                        if (g.accumulate) {
                            float old[4];
                            unpack4(*reinterpret_cast<const uint2 *>(cell), old);
#pragma unroll
                            for (int j = 0; j < 4; ++j) v[j] += old[j];
                        }
                    }
                    *reinterpret_cast<uint2 *>(cell) = pack4(v[0], v[1], v[2], v[3]);
                }
            }
        }
        flush(pass == 0 ? Cb : (bf16_t *)g.C2);
    }
}

// Writes the operand sums of a weight-gradient block (see Frags::mma_part): colsum[e][i] (+)= sum over the
// expert's rows of operand column i.  SUM 1: every register of lane l < 32 holds the sum for row l of the wave's
// summed m-block (block wn of wave row wm); SUM 2: register 4q+j of a lane holds the sum for column
// 8q + 4 (lane/32) + j of the wave's summed n-block (block wm of wave column wn).
template <int SUM, int C>
__device__ __forceinline__ void store_sums(const GemmArgs &g, const f32x16 &sums, int e, int m0, int n0, int m_ext, int wm,
                                           int wn, int lane) {
    bf16_t *out = (bf16_t *)g.colsum;
    if constexpr (SUM == 1) {
        const int m = m0 + (wm * C + wn) * 32 + (lane & 31);
        if (lane < 32 && wn < C && m < m_ext) {
            bf16_t *p = out + (long)e * g.M + m;
            float v = sums[0];
            if (g.accumulate) v += (float)*p;
            *p = (bf16_t)v;
        }
    } else {
        if ((lane & 31) == 0) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int n = n0 + wn * 64 + wm * 32 + 8 * q + 4 * (lane >> 5) + j;
                    if (n < g.N) {
                        bf16_t *p = out + (long)e * g.N + n;
                        float v = sums[4 * q + j];
                        if (g.accumulate) v += (float)*p;
                        *p = (bf16_t)v;
                    }
                }
        }
    }
}

// Row-ragged (!WG): C[rows_e, N] = Mop[rows_e, K] . Nop_e ; Mop K-contiguous, Nop_e [N,K] or (N_KS) [K,N].
// Weight gradient (WG): C_e[M, N] = sum_{r in rows_e} Mop[r, M]^T . Nop[r, N], both K-strided.
template <int TMB, int WM, bool N_KS, bool WG, int EPI>
__global__ __launch_bounds__((Tile<TMB, WM>::THREADS), (Tile<TMB, WM>::BLOCKS_PER_CU)) void gemm256_kernel(const GemmArgs g) {
    typedef Tile<TMB, WM> TL;
    constexpr bool M_KS = WG;
    constexpr int Q_BM = TL::BM, TMW = TL::TMW;
    extern __shared__ __align__(16) char smem[];
    // ---- which tile am I?  Blocks are dealt round-robin to the 8 XCDs (block b runs on XCD b mod 8):
    //      give each XCD a contiguous range of the REAL tiles, so that neighbours share operands in
    //      its L2 and every XCD gets the same share.  For row-ragged products the number of real
    //      tiles is only known here (the grid is sized for the worst case), hence the device-side sum.
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_tiles = (g.N + Q_BN - 1) / Q_BN;
    int sum_nt = 0, sum_mt = 0;   // weight gradients: the n-tile / m-tile whose block also sums the m-side / n-side operand
    int e, mt, nt, m_ext, k_ext, tile_h = Q_BM;   // tile_h: rows of this tile's m-tiles (row-ragged products cut experts evenly)
    long row0;  // first row of the expert
    if constexpr (!WG) {
        // An expert with r rows is cut into t = ceil(r / BM) m-tiles.  Where a launch is a single round of
        // tiles (the 320-row configuration of the two K = F products) they have equal height h = r / t
        // rounded up to whole 32-row blocks, so that no expert leaves a short remainder tile behind, which
        // would run as a second, nearly empty round; elsewhere they are BM rows high and the last one is
        // the remainder, which costs fewer MFMA blocks in total and fills in among the many rounds.  The
        // m-tiles of all experts are numbered in expert order and each XCD takes a contiguous range of the
        // real (m-tile, n-tile) pairs, so that neighbours share operands in its L2 and every XCD gets the
        // same share; their number is only known here (the grid is sized for the worst case).
        const bool single = g.offsets == nullptr;
        auto rows_of = [&](int ee) { return single ? g.single_rows : g.kept[ee]; };
        const int nE = single ? 1 : g.E;
        // rows and first row of the first 256 experts, fetched together (lane l holds experts l, l + 64, l + 128,
        // l + 192): the lookups below then need no further loads.  Fetched where they were needed, each pass of the
        // search below and the two lookups after it waited for memory in turn - four to five dependent round trips
        // per tile for experts past the 64th, half of a tile's fixed cost with 256 experts and a contraction of 1024.
        // (Beyond 256 experts the rest is read through the cache as before.)
        constexpr int RC = 4;
        int rows_c[RC], off_c[RC];
#pragma unroll
        for (int c = 0; c < RC; ++c) {
            const int ee = lane + WAVE * c;
            rows_c[c] = ee < nE ? rows_of(min(ee, nE - 1)) : 0;
            off_c[c] = (!single && ee < nE) ? g.offsets[min(ee, nE - 1)] : 0;
        }
        auto rows_at = [&](int ee) {            // rows of expert ee = base + lane of the caller's pass (ee uniform in ee / 64)
            int r = 0;
#pragma unroll
            for (int c = 0; c < RC; ++c)
                if ((ee >> 6) == c) r = rows_c[c];
            return (ee >> 6) < RC ? r : (ee < nE ? rows_of(ee) : 0);
        };
        // An expert's m-tiles are heavy (more than half a tile of rows) or light: the full tiles and, of the
        // remainder scheme, a remainder above half a tile; with the even split all tiles of an expert alike.
        // Heavy tiles are numbered before light ones, each class in expert order and each XCD taking a contiguous
        // range of either: an XCD hands out its blocks in order, so the long tiles start first and the short
        // ones fill in behind them (otherwise a long tile that starts late ends the launch late).
        // That order runs an expert's light tile long after its heavy ones, whose weight panels have left the L2 by
        // then; with many rounds of tiles the order matters little and the re-read does, so beyond 16 rounds
        // all tiles count as one class, in expert order.
        auto tiles_of = [&](int r) { return (r + Q_BM - 1) / Q_BM; };     // m-tiles of an expert with r rows
        bool split = true;
        auto heavy_of = [&](int r) {
            const int cnt = tiles_of(r);
            if (cnt == 0 || !split) return cnt;
            if (TMB == 10) return ((((r + cnt - 1) / cnt) + 31) & ~31) > Q_BM / 2 ? cnt : 0;
            return cnt - 1 + ((r - (cnt - 1) * Q_BM) > Q_BM / 2 ? 1 : 0);
        };
        int n_h = 0, n_l = 0;
        for (int ee = lane; ee < nE; ee += WAVE) {
            const int r = rows_at(ee);
            const int hv = heavy_of(r);
            n_h += hv;
            n_l += tiles_of(r) - hv;
        }
        for (int d = WAVE / 2; d >= 1; d >>= 1) { n_h += __shfl_xor(n_h, d, WAVE); n_l += __shfl_xor(n_l, d, WAVE); }
        if ((n_h + n_l) * n_tiles > 16 * 256) { split = false; n_h += n_l; n_l = 0; }
        const int total_h = n_h * n_tiles, total_l = n_l * n_tiles;
        const int per_h = (total_h + 7) >> 3, per_l = (total_l + 7) >> 3;
        const int slot = blockIdx.x >> 3, xcd = blockIdx.x & 7;
        const bool heavy = slot < per_h;
        const int t = heavy ? xcd * per_h + slot : xcd * per_l + (slot - per_h);
        if (heavy ? t >= total_h : (slot - per_h >= per_l || t >= total_l)) return;
        // Order of an XCD's tiles.  n-tile first: tile t = (m-tile t / n_tiles, n-tile t % n_tiles); the blocks that
        // run side by side on an XCD are then a few m-tiles times all n-tiles, i.e. they stream the expert's whole
        // weight matrix through the L2 once per group of m-tiles.  m-tile first (m_fastest): an expert's tiles are
        // numbered n-tile by n-tile, all its m-tiles of the class inside; the blocks side by side are then all
        // m-tiles of the expert times a few n-tiles, and every weight panel is fetched once.  In between (m_fastest =
        // G > 1): groups of G n-tiles with the expert's m-tiles inside, so that the 32 blocks of an XCD are about
        // 32 / G m-tiles times G n-tiles and fetch 32 / G + G panels between them instead of 1 + 32.  The two products
        // with a contraction over M and wide results (h = xd.w1^T + b1, t = (go.w2^T) gelu'(h)) use G = 8 for experts
        // of at least m_fastest_from = 8 m-tiles (8192 tokens, 64 experts of 2048 -> 8192, top-2, skewed loads: 798 ->
        // 766 and 777 -> 752 us); for experts of four or five m-tiles it is the slower order (16 experts of about 1024
        // rows, 1024 -> 4096: +6 and +3 us), so those keep n-tile first.
        const bool mf = g.m_fastest != 0;
        const int unit = mf ? n_tiles : 1;       // tiles per counted m-tile
        const int target = mf ? t : t / n_tiles;
        nt = t % n_tiles;
        // the expert whose running count (of the class) passes `target`
        int run = 0, found = -1, before = 0, cnt_found = 1;
        for (int base = 0; base < nE && found < 0; base += WAVE) {
            const int ee = base + lane;
            const int r = rows_at(ee);
            const int hv = heavy_of(r);
            const int cnt = (heavy ? hv : tiles_of(r) - hv) * unit;
            int incl = cnt;
            for (int d = 1; d < WAVE; d <<= 1) {
                const int y = __shfl_up(incl, d, WAVE);
                if (lane >= d) incl += y;
            }
            const unsigned long long hit = __ballot(run + incl > target);
            if (hit) {
                const int src = __ffsll(hit) - 1;
                found = base + src;
                before = run + __shfl(incl - cnt, src, WAVE);
                cnt_found = __shfl(cnt, src, WAVE);
            }
            run += __shfl(incl, WAVE - 1, WAVE);
        }
        if (found < 0) return;
        e = found;
        // (found is the same in every lane: the expert's chunk register, then the lane that holds it)
        {
            int mv = 0;
#pragma unroll
            for (int c = 0; c < RC; ++c)
                if ((found >> 6) == c) mv = __shfl(rows_c[c], found & 63, WAVE);
            m_ext = (found >> 6) < RC ? mv : rows_of(e);
        }
        int mt_class = target - before;
        if (mf && cnt_found / n_tiles < g.m_fastest_from) {
            // an expert with few m-tiles keeps the n-tile-first order (its tiles are counted one by one here)
            nt = mt_class % n_tiles;
            mt_class /= n_tiles;
        } else if (mf) {
            // groups of G n-tiles, an expert's m-tiles of the class inside a group, the group's n-tiles innermost
            // (G = 1: m-tile first; the last group may be short)
            const int c_e = cnt_found / n_tiles;      // the expert's m-tiles of this class
            const int G = g.m_fastest;
            const int n_groups = (n_tiles + G - 1) / G;
            const int grp = min(mt_class / (c_e * G), n_groups - 1);
            const int j = mt_class - grp * c_e * G;
            const int gsz = min(G, n_tiles - grp * G);
            nt = grp * G + j % gsz;
            mt_class = j / gsz;
        }
        mt = mt_class + (heavy ? 0 : heavy_of(m_ext));   // an expert's light tiles follow its heavy ones
        const int t_e = (m_ext + Q_BM - 1) / Q_BM;
        tile_h = TMB == 10 ? ((((m_ext + t_e - 1) / t_e) + 31) & ~31) : Q_BM;
        {
            int ov = 0;
#pragma unroll
            for (int c = 0; c < RC; ++c)
                if ((found >> 6) == c) ov = __shfl(off_c[c], found & 63, WAVE);
            row0 = single ? 0 : ((found >> 6) < RC ? ov : g.offsets[e]);
        }
        k_ext = g.K;
    } else {
        // The contraction length differs from expert to expert, so experts are not handed to XCDs in
        // contiguous ranges: the (expert, m-tile) units are dealt round-robin over the 8 XCDs, which gives
        // every XCD the same share of every expert; the n-tiles of a unit stay together (they share the
        // m-side operand in that XCD's L2).
        // With hundreds of experts of similar size that spread is not needed, and it costs traffic: the m-tiles of
        // an expert on different XCDs each fetch the expert's rows of the n-side operand into their own L2 (3x the
        // operands' bytes at 256 experts, which made the launch HBM-bound).  Then (wg_expert_major) the experts are
        // dealt round-robin instead, all blocks of one expert on one XCD.
        const int m_tiles = (g.M + Q_BM - 1) / Q_BM;
        const int slot = blockIdx.x >> 3;
        if (g.wg_expert_major) {
            const int u = slot / n_tiles;
            e = (u / m_tiles) * 8 + (blockIdx.x & 7);
            mt = u % m_tiles;
            if (e >= g.E) return;
        } else {
            const int unit = (slot / n_tiles) * 8 + (blockIdx.x & 7);
            if (unit >= g.E * m_tiles) return;
            e = unit / m_tiles;
            mt = unit % m_tiles;
        }
        nt = slot % n_tiles;
        // Blocks that also sum an operand run an eighth longer.  Consecutive slots of an XCD go to its four
        // shader engines in turn and are handed out in order, so an engine that always gets the long blocks
        // holds up the other three: the summing n-tile moves on from unit to unit, which gives every engine the
        // same number of long blocks in every round; the summing m-tile moves on from expert to expert, which
        // spreads those blocks over the XCDs.
        sum_nt = (slot / n_tiles) % n_tiles;
        sum_mt = e % m_tiles;
        m_ext = g.M;
        k_ext = g.kept ? g.kept[e] : g.single_rows;
        row0 = g.offsets ? g.offsets[e] : 0;
    }
    // the tile's coordinates are the same in every lane: say so, so that everything derived from them
    // (operand bases, LDS destinations, loop bounds) lives in scalar registers
    e = __builtin_amdgcn_readfirstlane(e);
    mt = __builtin_amdgcn_readfirstlane(mt);
    tile_h = __builtin_amdgcn_readfirstlane(tile_h);
    nt = __builtin_amdgcn_readfirstlane(nt);
    sum_nt = __builtin_amdgcn_readfirstlane(sum_nt);
    sum_mt = __builtin_amdgcn_readfirstlane(sum_mt);
    m_ext = __builtin_amdgcn_readfirstlane(m_ext);
    k_ext = __builtin_amdgcn_readfirstlane(k_ext);
    row0 = ((long)__builtin_amdgcn_readfirstlane((int)(row0 >> 32)) << 32) | (unsigned)__builtin_amdgcn_readfirstlane((int)row0);
    const int m0 = mt * tile_h, n0 = nt * Q_BN;
    if constexpr (WG && EPI == EPI_WGRAD) {
        if (k_ext == 0) {
            // An expert without rows: its gradient tile is zero (and adds nothing when sums are being built up).  The
            // zeros leave straight from registers, two 512-byte row pieces per wave and store - no operand ring, no
            // LDS slab, no barrier (with skewed loads most experts of a launch are such: 28 of 64 at 8192 tokens,
            // top-2, Zipf(1.2)).
            if (g.accumulate) return;
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            bf16_t *Cz = (bf16_t *)g.C + (long)e * g.strideC;
            const int col = n0 + (lane & 31) * 8;
            for (int r = wave * 2 + (lane >> 5); r < Q_BM; r += 2 * TL::NW) {
                const int m = m0 + r;
                if (m < m_ext && col < g.N)
                    __builtin_nontemporal_store(u32x4{0u, 0u, 0u, 0u}, reinterpret_cast<u32x4 *>(Cz + (long)m * g.ldc + col));
            }
            if (g.colsum != nullptr) {
                bf16_t *out = (bf16_t *)g.colsum;
                const bf16_t z = (bf16_t)0.0f;
                if (g.colsum_side == 1 && nt == sum_nt) {
                    for (int r = threadIdx.x; r < Q_BM; r += TL::THREADS)
                        if (m0 + r < m_ext) out[(long)e * g.M + m0 + r] = z;
                } else if (g.colsum_side == 2 && mt == sum_mt) {
                    for (int c = threadIdx.x; c < Q_BN; c += TL::THREADS)
                        if (n0 + c < g.N) out[(long)e * g.N + n0 + c] = z;
                }
            }
            return;
        }
    }
    const bf16_t *Mp = (const bf16_t *)g.A + row0 * g.lda;
    const bf16_t *Np = WG ? (const bf16_t *)g.B + row0 * g.ldb : (const bf16_t *)g.B + (long)e * g.strideB;

    f32x16 acc[TMW][2];
#pragma unroll
    for (int i = 0; i < TMW; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

    const int live = min(tile_h, m_ext - m0);
    const int tmc = (live + 31) >> 5;
    const int wu = __builtin_amdgcn_readfirstlane(wave);
    const int wm = WM == 1 ? 0 : wu >> 2, wn = wu & 3;     // wave row / wave column
    uint2 bias_raw[8];
    load_bias<EPI>(g, e, n0, lane, wn, bias_raw);
    // Operand sums ride along in the weight-gradient blocks that see the whole operand once: one n-tile
    // of every m-tile for the m-side, one m-tile of every n-tile for the n-side.  These blocks run the
    // full tile shape (blocks past the operand's end repeat its last row and are not stored).
    int sum_side = 0;
    if constexpr (WG && WM == 2 && TMW == 4) {
        if (g.colsum != nullptr && ((g.colsum_side == 1 && nt == sum_nt) || (g.colsum_side == 2 && mt == sum_mt))) sum_side = g.colsum_side;
    }
    // The live blocks are dealt evenly to the wave rows: c to each (the last row may find fewer live).
    const int c = sum_side ? TMW : (tmc + WM - 1) / WM;
    const int m0w = m0 + wm * c * 32, live_w = max(0, min(live - wm * c * 32, c * 32));
    // K loop and epilogue with C blocks per wave row
    f32x16 sums;
#pragma unroll
    for (int q = 0; q < 16; ++q) sums[q] = 0.f;
#define MOLE_RUN_TILE_SUM(C, SUM)                                                                                         \
    {                                                                                                                     \
        main_loop<TMB, WM, M_KS, N_KS, WG, WM *(C), (C), SUM, (EPI > EPI_NONE ? EPI - EPI_NONE : 0), (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU)>(Mp, g.lda, m0, m_ext, Np, g.ldb, n0, g.N, k_ext, smem, wu, wm, wn, acc, sums, bias_raw); \
        if constexpr (SUM != 0) store_sums<SUM, (C)>(g, sums, e, m0, n0, m_ext, wm, wn, lane);                            \
        epilogue<TMB, WM, WG, EPI, (C)>(g, acc, smem, lane, wu, wn, e, row0, m0w, n0, m_ext, live_w, bias_raw);      \
    }
#define MOLE_RUN_TILE(C) MOLE_RUN_TILE_SUM(C, 0)
    if constexpr (WG && WM == 2 && TMW == 4) {
        if (sum_side == 1) { MOLE_RUN_TILE_SUM(TMW, 1) return; }
        if (sum_side == 2) { MOLE_RUN_TILE_SUM(TMW, 2) return; }
    }
    if constexpr (WM == 1) {
        if (c > TMB / 2) MOLE_RUN_TILE(TMB)
        else if (c > TMB / 4) MOLE_RUN_TILE(TMB / 2)
        else MOLE_RUN_TILE(TMB / 4)
    } else {
        if (c >= TMW) MOLE_RUN_TILE(TMW)
        else if (TMW > 4 && c == 4) MOLE_RUN_TILE(TMW > 4 ? 4 : 1)
        else if (c == 3) MOLE_RUN_TILE(3)
        else if (c == 2) MOLE_RUN_TILE(2)
        else MOLE_RUN_TILE(1)
    }
#undef MOLE_RUN_TILE
#undef MOLE_RUN_TILE_SUM
}

template <int TMB, int WM, bool N_KS, bool WG, int EPI>
static int launch256(GemmArgs g, int tiles, hipStream_t st, int kid) {
    typedef Tile<TMB, WM> TL;
    if (tiles <= 0) return 0;
    g.n_blocks = tiles;
    const int grid = (tiles + 7) & ~7;
    auto kern = gemm256_kernel<TMB, WM, N_KS, WG, EPI>;
    static bool attr_done = false;
    if (!attr_done) {
        MOLE_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, TL::LDS_BYTES));
        attr_done = true;
    }
    timed_launch(kid, kern, dim3(grid), dim3(TL::THREADS), TL::LDS_BYTES, st, g);
    MOLE_LAUNCH_CHECK();
    return 0;
}

// Launch options and their defaults; a -DMOLE_TUNING build reads them from the environment
// (MOLE_MFAST: bit mask of the products that number an expert's tiles m-tile first within groups of MOLE_MFAST_G
// n-tiles, MOLE_MFAST_FROM: m-tiles an expert needs for that order, MOLE_WG_EMAJOR: expert count from which a weight gradient keeps an expert's blocks on one XCD,
// MOLE_TMB: 4 | 8 = four-wave tiles of 128 | 256 rows, 16 = the 256-row eight-wave tile for every product,
// MOLE_NO_SUMS: bias gradients from their own kernel).
#ifdef MOLE_TUNING
static int env_int(const char *name, int dflt) { const char *v = getenv(name); return v ? atoi(v) : dflt; }
static int m_fastest_mask() { static const int v = env_int("MOLE_MFAST", 9); return v; }
static int m_fastest_group() { static const int v = env_int("MOLE_MFAST_G", 8); return v > 0 ? v : 1; }
static int m_fastest_from() { static const int v = env_int("MOLE_MFAST_FROM", 8); return v; }
static int wg_emajor_from() { static const int v = env_int("MOLE_WG_EMAJOR", 128); return v; }
static int forced_tile() { static const int v = env_int("MOLE_TMB", 0); return v; }
static bool sums_off() { static const bool v = getenv("MOLE_NO_SUMS") != nullptr; return v; }
#else
static int m_fastest_mask() { return 9; }        // h = xd.w1^T + b1 and t = (go.w2^T) gelu'(h)
static int m_fastest_group() { return 8; }
static int m_fastest_from() { return 8; }
static int wg_emajor_from() { return 128; }
static int forced_tile() { return 0; }
static bool sums_off() { return false; }
#endif

template <int TMB, int WM>
static int dispatch256(const GemmArgs &g, bool b_ks, bool wg, int epi, int max_rows, hipStream_t st, int kid) {
    constexpr int BM = Tile<TMB, WM>::BM;
    const int n_tiles = ceil_div(g.N, Q_BN);
    if constexpr (TMB != 10) {
        if (wg) {
            GemmArgs gw = g;
            gw.wg_expert_major = g.E >= wg_emajor_from();
            // whole (expert, m-tile) units per XCD, or whole experts
            const int tiles = gw.wg_expert_major ? 8 * ceil_div(g.E, 8) * ceil_div(g.M, BM) * n_tiles
                                                 : 8 * ceil_div(g.E * ceil_div(g.M, BM), 8) * n_tiles;
            if (epi == EPI_WGRAD) return launch256<TMB, WM, true, true, EPI_WGRAD>(gw, tiles, st, kid);
            return -100;
        }
    }
    // block slots: the worst-case number of m-tiles (an expert with r rows has ceil(r / BM) of them)
    const int rows_bound = g.offsets ? max_rows : g.single_rows;
    GemmArgs gg = g;
    gg.m_fastest = ((m_fastest_mask() >> kid) & 1) ? m_fastest_group() : 0;
    gg.m_fastest_from = m_fastest_from();
    // (+ 16: the heavy and the light tiles of an XCD are rounded up to whole slots separately)
    const int tiles = (((rows_bound / BM + (g.offsets ? g.E : 1)) * n_tiles + 7) & ~7) + 16;
    if (wg) return -100;
    if (!b_ks) {
        if constexpr (TMB != 10) {
            if (epi == EPI_DGELU) return launch256<TMB, WM, false, false, EPI_DGELU>(gg, tiles, st, kid);
            if (epi == EPI_BIAS_GELU) return launch256<TMB, WM, false, false, EPI_BIAS_GELU>(gg, tiles, st, kid);
            if (epi == EPI_F32) return launch256<TMB, WM, false, false, EPI_F32>(gg, tiles, st, kid);
            if (epi == EPI_NONE) return launch256<TMB, WM, false, false, EPI_NONE>(gg, tiles, st, kid);
#ifdef MOLE_TUNING
            if constexpr (TMB == 8 && WM == 2) {     // the loop's parts are probed at the default tile shape only
                if (epi == EPI_NONE + 1) return launch256<TMB, WM, false, false, EPI_NONE + 1>(gg, tiles, st, kid);
                if (epi == EPI_NONE + 2) return launch256<TMB, WM, false, false, EPI_NONE + 2>(gg, tiles, st, kid);
                if (epi == EPI_NONE + 3) return launch256<TMB, WM, false, false, EPI_NONE + 3>(gg, tiles, st, kid);
                if (epi == EPI_NONE + 4) return launch256<TMB, WM, false, false, EPI_NONE + 4>(gg, tiles, st, kid);
            }
#endif
        }
    } else {
        if (epi == EPI_BIAS) return launch256<TMB, WM, true, false, EPI_BIAS>(gg, tiles, st, kid);
        if (epi == EPI_STORE) return launch256<TMB, WM, true, false, EPI_STORE>(gg, tiles, st, kid);
    }
    return -100;
}

// Tile configuration.  Eight waves (two per SIMD hide each other's waits; one fetch of the n-side tile
// serves all rows of the tile) for every product.  256-row tiles by default; tiles of up to 320 rows, an
// expert's rows split evenly over them, for the two K = F products (out = a.w2 + b2 and gx = t.w1): one tile
// is a whole round there, and with a capacity factor of 1.25 no expert then needs more m-tiles than the
// average one, so the launch stays one round.  The K = M products run four rounds anyway; their short
// remainder tiles, numbered last, fill the final round, which measured better than the even split
// (t = (go.w2^T) gelu'(h): 213 against 219 us) - and h = xd.w1^T + b1 with the GELU epilogue would spill at
// the 160 accumulators of the larger tile.
static int tile_blocks_for(int kid) {
    const int forced = forced_tile();
    if (forced == 4 || forced == 8 || forced == 16) return forced;
    return (kid == MOLE_K_FFN_FWD2 || kid == MOLE_K_FFN_GX) ? 20 : 16;
}

// Whether the weight-gradient launch for g will also produce the operand sums asked for in g.colsum
// (the eight-wave 256-row tile does; the tuning variants and the generic kernel do not).
bool gemm256_sums_operand(const GemmArgs &g, int kid) {
    if (g.lda % 8 || g.ldb % 8 || g.ldc % 8 || g.N % 8 || g.M % 8) return false;
    const int tmb = tile_blocks_for(kid);
    if (sums_off()) return false;
    return tmb == 16 || tmb == 20;
}

int launch_gemm256(const GemmArgs &g, bool a_ks, bool b_ks, bool wg, int epi, int max_rows, hipStream_t st, int kid) {
    // alignment the direct-to-LDS path relies on: 16-byte rows, whole stages of K for row-ragged products
    if (g.lda % 8 || g.ldb % 8 || g.ldc % 8 || g.N % 8) return -100;
    if (!wg && (a_ks || g.K % Q_BK)) return -100;
    if (wg && (!a_ks || !b_ks || g.M % 8)) return -100;
    const int tmb = tile_blocks_for(kid);
#ifdef MOLE_TUNING
    if (tmb == 4) return dispatch256<4, 1>(g, b_ks, wg, epi, max_rows, st, kid);
    if (tmb == 8) return dispatch256<8, 1>(g, b_ks, wg, epi, max_rows, st, kid);
#endif
    if (tmb == 20 && !wg && b_ks) return dispatch256<10, 2>(g, b_ks, wg, epi, max_rows, st, kid);   // up to 320 rows, eight waves
    return dispatch256<8, 2>(g, b_ks, wg, epi, max_rows, st, kid);                                  // 256 rows, eight waves
}

}  // namespace mole
