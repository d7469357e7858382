/*
 * mole_hip.h - C ABI of the MI355X (gfx950) MoE-layer hot path.
 *
 * This is the drop-in boundary for MOLE's single-GPU MoE layer.  Every entry point replaces a
 * piece of what the reference reaches through pybind (MOLE/cpp/core.cpp:1347-1469) or through
 * the third-party tutel package (MOLE/moe/layer.py:445-458).  Rules of the boundary:
 *
 *   - plain C: pointers, sizes, enums.  No C++ types, no torch types, no exceptions, no exit().
 *   - every function returns 0 on success, a positive hipError_t, or a negative MOLE_E_* code;
 *     mole_last_error_string() describes the last failure on the calling thread.
 *   - the caller allocates every buffer (inputs, outputs, saved activations, workspaces).  The
 *     library owns only what mole_unimem_create() makes: the slot pool, its copy stream and events.
 *   - all kernels are enqueued on the caller's stream (a hipStream_t passed as void*) and never
 *     synchronise the host; the only blocking calls are mole_unimem_sync_tran() and the
 *     create/destroy pair.
 *   - all tensors are dense row-major.  Row pointers of x/xd/o/h must be 16-byte aligned
 *     (M and F multiples of 8 for bf16, of 4 for fp32).
 *
 * Symbols: S tokens, M model dim (embed_dim), E experts, k top-k, F ffn dim, C capacity.
 */
#ifndef MOLE_HIP_H
#define MOLE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *mole_stream_t; /* a hipStream_t; NULL is the default stream */

enum { MOLE_F32 = 0, MOLE_BF16 = 1 };
/* where expert e's rows start: PADDED is the reference's [E, C, M] layout (row = e*C + loc),
 * RAGGED packs the kept rows of the experts back to back (row = offsets[e] + loc). */
enum { MOLE_LAYOUT_PADDED = 0, MOLE_LAYOUT_RAGGED = 1 };
/* derivative used for the GELU in the backward pass.  TANH is what the reference compiles
 * (MOLE/cpp/define.hpp:6 -> MOLE/cpp/gelu.cu:3-14); EXACT is the erf derivative
 * (at::gelu_backward, MOLE/cpp/core.cpp:396). */
enum { MOLE_GELU_BWD_TANH = 0, MOLE_GELU_BWD_EXACT = 1 };

enum {
    MOLE_E_INVALID = -1,   /* bad argument (null pointer, size out of range, misalignment) */
    MOLE_E_WORKSPACE = -2, /* workspace too small */
    MOLE_E_STATE = -3,     /* call does not fit the handle's state (e.g. pool exhausted) */
    MOLE_E_NOMEM = -4
};

#define MOLE_MAX_TOPK 16
#define MOLE_MAX_EXPERTS 1024

int mole_version(void);
const char *mole_last_error_string(void);

/* Optional per-kernel timing for benchmarks (no counterpart in the reference, whose timers wrap
 * whole layers: MOLE/utils/Utimer.py:5-70).  While enabled, each kernel launch carries a start and a
 * stop event of its own (entry points that launch several kernels under one id are bracketed by two
 * events on the stream instead); mole_kernel_timing_read() waits for them and returns, for ids
 * 0..n_ids-1, the number of launches and their summed duration in ms, then forgets them. */
enum {
    MOLE_K_FFN_FWD1 = 0,  /* h = xd.w1^T + b1, a = gelu(h) */
    MOLE_K_FFN_FWD2 = 1,  /* out = a.w2 + b2 */
    MOLE_K_FFN_GW2 = 2,   /* g_w2 = a^T.go */
    MOLE_K_FFN_DA = 3,    /* t = (go.w2^T) * gelu'(h) */
    MOLE_K_FFN_GW1 = 4,   /* g_w1 = t^T.xd */
    MOLE_K_FFN_GX = 5,    /* gx = t.w1 */
    MOLE_K_FFN_GB = 6,    /* bias gradients */
    MOLE_K_DISPATCH_FWD = 7,
    MOLE_K_DISPATCH_BWD = 8,
    MOLE_K_COMBINE_FWD = 9,
    MOLE_K_COMBINE_BWD = 10,
    MOLE_K_ROUTE = 11,    /* the four routing kernels together */
    MOLE_K_GEMM_NT = 12,
    MOLE_K_ADAM = 13,
    MOLE_K_GATE_FWD = 14,   /* gate logits + softmax in one kernel, or the softmax kernel alone */
    MOLE_K_GATE_BWD = 15,   /* dgates -> dlogits */
    MOLE_K_GATE_WGRAD = 16, /* dWg: partial sums + their reduction */
    MOLE_K_RESERVED_17 = 17, /* timing slot of the measurement aids declared in mole_hip_probe.h */
    MOLE_K_COUNT = 18
};
int mole_kernel_timing_enable(int on);
int mole_kernel_timing_read(int n_ids, int *counts, float *ms_total);

/* ------------------------------------------------------------------------------------------
 * Gate.  Replaces MOLETopk.forward (MOLE/utils/Ugate.py:11-14): scores = softmax(logits).
 * logits [S,E] fp32 (x . Wg^T, produced by mole_gemm_nt or any GEMM); logit_bias [E] or NULL.
 * mole_gate_bwd replaces the autograd of the gate normalisation inside tutel's
 * extract_critical and, with through_softmax != 0, of the softmax as well: from dgates [k,S]
 * it produces d(scores) [S,E] (through_softmax == 0) or d(logits) [S,E].  counts0 [E] (the first
 * choice's per-expert counts from mole_route) and d_l_aux [1] (device, the gradient arriving at l_aux) are
 * given together or both NULL: with them d(scores)[i,e] also carries d_l_aux * E/S^2 * counts0[e], the
 * gradient of tutel's gshard_loss, which the reference adds to its loss through autograd (MOLE/moe/layer.py:447).
 * ------------------------------------------------------------------------------------------ */
int mole_softmax_fwd(const float *logits, const float *logit_bias, int S, int E, float *scores,
                     mole_stream_t stream);
/* dlogits = scores * (dscores - sum_e dscores scores): the softmax's backward alone, for the gate module used
 * outside the fused layer (autograd runs it in the reference, MOLE/utils/Ugate.py:13). */
int mole_softmax_bwd(const float *dscores, const float *scores, int S, int E, float *dlogits,
                     mole_stream_t stream);
/* The whole of MOLETopk.forward (MOLE/utils/Ugate.py:11-14) in one kernel:
 * scores[S,E] = softmax(x[S,M] . wg[E,M]^T + logit_bias), wg fp32, logit_bias [E] or NULL.
 * bf16 tokens: M a multiple of 128, E <= 256; wg is rounded to bf16 for the products, fp32 accumulation.  Every
 * block of 16-64 tokens reads all of wg, so beyond 64 experts the two-kernel path is the faster one (the Python
 * host side switches there).
 * fp32 tokens: M a multiple of 4, E <= 32, x and wg 16-byte aligned; fp32 FMAs throughout.
 * Other cases use mole_gemm_nt + mole_softmax_fwd. */
int mole_gate_fwd(const void *x, int dtype, const float *wg, const float *logit_bias, int S, int E, int M,
                  float *scores, mole_stream_t stream);
int mole_gate_bwd(const float *dgates, const float *scores, const int32_t *idx, int S, int E,
                  int k, int normalize_gate, int through_softmax, const int32_t *counts0, const float *d_l_aux,
                  float *dout, mole_stream_t stream);
/* Gradient of the gate's Linear (MOLE/utils/Ugate.py:12, run by autograd in the reference):
 * dwg[E,M] = dlogits[S,E]^T . x[S,M], fp32, summed in a fixed order (partial sums per chunk of tokens in the
 * workspace, then a reduction).  bf16 tokens: E <= 256 and M a multiple of 64 on the matrix cores (dlogits
 * enters as the sum of two bf16 numbers, so the result keeps fp32-level accuracy); either dtype: E <= 32 and
 * M a multiple of 4 on the VALU.  Other shapes are rejected (a library GEMM serves them on the host side).
 * workspace of mole_gate_wgrad_workspace_bytes(S, E, M) bytes. */
size_t mole_gate_wgrad_workspace_bytes(int S, int E, int M);
int mole_gate_wgrad(const float *dlogits, const void *x, int dtype, int S, int E, int M, float *dwg,
                    void *workspace, size_t workspace_bytes, mole_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Routing.  Replaces tutel.impls.fast_dispatch.extract_critical (call site
 * MOLE/moe/layer.py:445-446): top-k with ties to the lowest expert index, gate values
 * (normalised over the k choices when k > 1 and normalize_gate), per-choice per-expert counts,
 * k-major locations, capacity, and the dispatch permutation.
 *
 *   scores   [S,E] fp32 in
 *   idx      [k,S] int32 out   chosen expert of every (choice, token)
 *   loc      [k,S] int32 out   location inside the expert (before the capacity test)
 *   gates    [k,S] fp32  out
 *   row      [k,S] int32 out   destination row in the dispatched buffer, -1 when dropped
 *   counts   [k,E] int32 out
 *   kept_rows[E]   int32 out   n[e] = min(sum_j counts[j,e], C)
 *   offsets  [E+1] int32 out   first row of expert e (RAGGED: prefix sum of kept_rows,
 *                              PADDED: e*C); offsets[E] = total rows
 *   capacity [1]   int32 out   C, on the device (capacity_factor <= 0 makes it data dependent)
 *   l_aux    [1]   fp32  out   E/S^2 * sum_e (sum_i scores[i,e]) * counts[0,e]; may be NULL
 *
 * capacity_factor > 0: C = k*int(cf*ceil(S/E)); == 0: C = max(loc)+1; < 0: the smaller of both;
 * C is then rounded up to `alignment`.  The factor is a double and the product is taken in double precision,
 * like the Python expression it replaces (0.02 * 50 must give 1, which single precision does not).
 * k is clipped to E by the caller (k <= E required).
 * ------------------------------------------------------------------------------------------ */
size_t mole_route_workspace_bytes(int S, int E, int k);
int mole_route(const float *scores, int S, int E, int k, double capacity_factor, int normalize_gate,
               int alignment, int layout, int32_t *idx, int32_t *loc, float *gates, int32_t *row,
               int32_t *counts, int32_t *kept_rows, int32_t *offsets, int32_t *capacity,
               float *l_aux, void *workspace, size_t workspace_bytes, mole_stream_t stream);

/* mole_gate_fwd and mole_route in one call for small gates on bf16 tokens (E <= 64, M a multiple of 128, S >= 1): the gate
 * kernel goes on to the routing's first stage - top-k, gate values, in-block ranks, histograms - while a token's
 * scores are still in the lanes that formed them, so the routing starts one kernel later and never reads the scores
 * back (MOLE/utils/Ugate.py:11-14 followed by extract_critical, MOLE/moe/layer.py:442-446).  Arguments and results are
 * those of the two calls; scores [S,E] is an output here.  Every result equals the two calls' bit for bit except
 * l_aux, whose column sums are added in another order (32 tokens per block instead of 64).  Other shapes are rejected:
 * the caller runs the two calls. */
size_t mole_gate_route_workspace_bytes(int S, int E, int k);
int mole_gate_route(const void *x, int dtype, const float *wg, const float *logit_bias, int S, int E, int M, int k,
                    double capacity_factor, int normalize_gate, int alignment, int layout, float *scores,
                    int32_t *idx, int32_t *loc, float *gates, int32_t *row, int32_t *counts, int32_t *kept_rows,
                    int32_t *offsets, int32_t *capacity, float *l_aux, void *workspace, size_t workspace_bytes,
                    mole_stream_t stream);

/* mole_route for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the same routing with the same outputs, but without the workspace argument.
 * No counterpart in the reference.  The scratch the routing kernels need (per-block histograms, per-choice bases,
 * column sums of the scores) lives in a static device array of mole_route_static_max_bytes() = 8 MiB inside the
 * library, one copy per GPU, held until the process ends; the call allocates nothing, on the host side neither.
 * Problem sizes whose mole_route_workspace_bytes(S, E, k) exceeds the array are rejected with MOLE_E_WORKSPACE
 * (the five configurations of the benchmark set need at most 4.6 MiB).  All calls on one GPU share the array: calls that
 * overlap on one GPU (two streams, two threads) race on it and must be serialised by the caller.  The first
 * call on a device looks up the array's address (hipGetSymbolAddress) and must not run under stream capture. */
size_t mole_route_static_max_bytes(void);
int mole_route_static(const float *scores, int S, int E, int k, double capacity_factor, int normalize_gate,
                      int alignment, int layout, int32_t *idx, int32_t *loc, float *gates, int32_t *row,
                      int32_t *counts, int32_t *kept_rows, int32_t *offsets, int32_t *capacity,
                      float *l_aux, mole_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Dispatch / combine.  Replace tutel fast_encode / fast_decode and their backward
 * (call sites MOLE/moe/layer.py:448-449, 457-458).  `row` is mole_route's permutation.
 *
 *   dispatch_fwd : xd[row[j,i],:] = x[i,:]                      for kept pairs
 *   dispatch_bwd : dx[i,:] = sum_j dxd[row[j,i],:]  (+ dlogits[i,:] . Wg  when dlogits != NULL,
 *                  the gate's contribution to the input gradient, Wg [E,M] fp32)
 *                  (+ dx_add[i,:] when dx_add != NULL: the same contribution computed beforehand)
 *   combine_fwd  : y[i,:] = sum_j gates[j,i] * o[row[j,i],:]    (zeros for a fully dropped token)
 *   combine_bwd  : d_o[row[j,i],:] = gates[j,i]*dy[i,:];  dgates[j,i] = <dy[i,:], o[row[j,i],:]>
 *                  (0 for dropped pairs)
 *   zero_pad_rows: zero the rows of a [total_rows, M] buffer that no kept pair owns
 *                  (rows offsets[e]+kept_rows[e] .. offsets[e+1]), which the reference's zeroed
 *                  [E,C,M] buffers contain.
 * The expert-contiguous buffers (xd, dxd, o, d_o) must hold at least one row even when every pair was
 * dropped: the gathers read row 0 in place of a dropped pair's row and discard what they read.
 * The kernels are compiled for k <= 1, 2, 4, 8 and 16 and run the smallest that holds k.
 * ------------------------------------------------------------------------------------------ */
int mole_dispatch_fwd(const void *x, int dtype, const int32_t *row, int S, int M, int k, void *xd,
                      mole_stream_t stream);
int mole_dispatch_bwd(const void *dxd, int dtype, const int32_t *row, int S, int M, int k,
                      const float *dlogits, const float *wg, int E, const void *dx_add, void *dx,
                      mole_stream_t stream);
int mole_combine_fwd(const void *o, int dtype, const int32_t *row, const float *gates, int S,
                     int M, int k, void *y, mole_stream_t stream);
int mole_combine_bwd(const void *dy, const void *o, int dtype, const int32_t *row,
                     const float *gates, int S, int M, int k, void *d_o, float *dgates,
                     mole_stream_t stream);
/* mole_combine_bwd followed by mole_gate_bwd (below) in one kernel, for gates of up to 256 experts: the backward of
 * tutel's fast_decode (MOLE/moe/layer.py:457-458) and the autograd of the gate values inside extract_critical
 * (layer.py:445-446) and of the softmax (MOLE/utils/Ugate.py:11-14).  The k gate gradients of a token stay in the
 * wave that formed them; the arguments after d_o are those of mole_gate_bwd, dlogits [S,E] its result. */
int mole_combine_bwd_gate(const void *dy, const void *o, int dtype, const int32_t *row, const float *gates,
                          int S, int M, int k, void *d_o, const float *scores, const int32_t *idx, int E,
                          int normalize_gate, int through_softmax, const int32_t *counts0,
                          const float *d_l_aux, float *dlogits, mole_stream_t stream);
int mole_zero_pad_rows(void *buf, int dtype, const int32_t *kept_rows, const int32_t *offsets,
                       int E, int M, mole_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Grouped expert FFN.  Replaces _BatchRecord::bffn_fwd / bffn_bwd / bffn_bwd_acc
 * (MOLE/cpp/core.cpp:344-356, 381-414, 457-491) and the GELU-backward kernel
 * (MOLE/cpp/gelu.cu:16-58), with bias, GELU and GELU' fused into the GEMM epilogues.
 *
 * Expert e owns rows offsets[e] .. offsets[e]+kept_rows[e] of every [rows, *] buffer; both
 * arrays live on the device.  max_rows bounds offsets[e]+kept_rows[e] (it sizes the launch).
 *   w1 [E,F,M]  b1 [E,F]  w2 [E,F,M] (used as a . w2)  b2 [E,M]         (dtype)
 *   fwd: h = xd.w1^T + b1 ; a = gelu_erf(h) ; out = a.w2 + b2             h,a [rows,F]  out [rows,M]
 *   bwd: g_w2 = a^T.go ; t = (go.w2^T) * gelu'(h) ; g_b2 = sum go ; g_w1 = t^T.xd ;
 *        g_b1 = sum t ; gx = t.w1     (t [rows,F] is caller-provided scratch; gx may be NULL)
 *        accumulate != 0 adds into g_* instead of overwriting (bffn_bwd_acc).
 * fp32 accumulation throughout; bf16 buffers are rounded once, on store.
 * ------------------------------------------------------------------------------------------ */
int mole_ffn_fwd(const void *xd, int dtype, const int32_t *offsets, const int32_t *kept_rows, int E,
                 int max_rows, int M, int F, const void *w1, const void *b1, const void *w2,
                 const void *b2, void *h, void *a, void *out, mole_stream_t stream);
int mole_ffn_bwd(const void *go, const void *xd, const void *h, const void *a, int dtype,
                 const int32_t *offsets, const int32_t *kept_rows, int E, int max_rows, int M, int F,
                 const void *w1, const void *w2, void *t, void *g_w1, void *g_b1, void *g_w2,
                 void *g_b2, void *gx, int accumulate, int gelu_bwd, mole_stream_t stream);

/* Plain GEMMs on the same tiles, used by the gate: c[rows,N] = a[rows,K] . b[N,K]^T  (fp32 out). */
int mole_gemm_nt(const void *a, const void *b, int dtype, int rows, int N, int K, float *c,
                 mole_stream_t stream);
/* c[rows,N] = a[rows,K] . b[K,N], result in `dtype` (the gate's input gradient dlogits . Wg for gates
 * too large for mole_dispatch_bwd to fold in). */
int mole_gemm_nn(const void *a, const void *b, int dtype, int rows, int N, int K, void *c,
                 mole_stream_t stream);
/* c[Mo,N] = a[rows,Mo]^T . b[rows,N], result in `dtype`: the gate's weight gradient dlogits^T . x for the shapes
 * mole_gate_wgrad does not take (one output tile per block, the contraction over all rows inside it). */
int mole_gemm_tn(const void *a, const void *b, int dtype, int rows, int Mo, int N, void *c,
                 mole_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Slot pool and pinned-host expert prefetch.  Replaces _UniMem (MOLE/cpp/umemory.cpp,
 * MOLE/cpp/define.hpp:143-193), _CPUParamCore::prefetch_to (MOLE/cpp/uparameter.cpp:58-63),
 * _MOLECore::prefetch_fwd/bwd (MOLE/cpp/core.cpp:41-75), _BatchRecord::fetch_para
 * (MOLE/cpp/core.cpp:110-143), the H2D copies (MOLE/cpp/transfer.cu:9-12) and the stream/event
 * plumbing (MOLE/cpp/stream.cpp:38-55, 156-205).
 *
 * The pool holds pool_size expert slots for each of the four parameter kinds
 * p_id 0..3 = w1 [F,M], b1 [F], w2 [F,M], b2 [M].  host_src[p] points at expert `0` of the
 * pinned host array of kind p ([n_d, ...] contiguous); experts [base, base+n) are copied.
 *
 *   prefetch(layer, base, n)      reserve n slots at the virtual offset, push (layer, n) on the
 *                                 prefetch stack, copy on the library's copy stream, record the
 *                                 "parameters landed" event.
 *   fetch_top(layer)              pop the stack when its top belongs to `layer`; returns the number
 *                                 of experts already prefetched (0 if none) in *n_out.
 *   fetch(view_base, base, n, prefetched)
 *                                 make experts [base, base+n) resident in slots
 *                                 view_base+virtual_offset .. : waits for the last compute that
 *                                 used those slots, copies the part not yet prefetched, records the
 *                                 event.
 *   wait_params(stream)           the compute stream waits for every copy issued so far.
 *   wait_slots(view_base, n, stream)
 *                                 the compute stream waits for the experts in slots view_base+virtual_offset ..
 *                                 only (each expert carries an event of its own): a chunk starts computing
 *                                 while the rest of a large prefetch is still arriving.
 *   release(view_base, n, stream) records that compute on `stream` has finished with the slots.
 *
 * prefetch_ids / fetch_ids are the same two calls for an explicit list of experts instead of a range:
 * expert expert_ids[i] (an index into the pinned host arrays; the library checks ids for >= 0 only - it is handed
 * base pointers, not extents, so the caller guarantees that every id, like every base + n of the range forms,
 * lies inside its host arrays, as the reference's callers do for their tensor slices) lands in the i-th slot of the call, so the
 * host side can bring in only the experts that routing activated (kept_rows[e] > 0) and hand the grouped
 * FFN a compacted offsets / kept_rows pair in the same order.  The reference always copies whole index
 * ranges (MOLE/cpp/core.cpp:41-57, 1025-1047); these two have no counterpart there.  Consecutive ids that
 * `tag` (0: none) lets a slot keep what it holds: a slot last filled under the same non-zero tag from the same
 * host expert is not copied again.  The caller vouches that the host arrays are unchanged since that copy; the
 * host side hands out one tag per forward pass of a layer and uses it again only for that pass's backward, so
 * that experts still resident from the forward are not fetched a second time (the reference always fetches
 * again, MOLE/cpp/core.cpp:1203).  mole_unimem_reuse_stats: bytes of the requests answered that way since the last
 * read (an expert asked for twice while in place counts twice).
 * ------------------------------------------------------------------------------------------ */
int mole_unimem_create(int device, int pool_size, int dtype, int64_t F, int64_t M, void **handle);
int mole_unimem_destroy(void *handle);
int mole_unimem_clear_virtual_mem(void *handle);
int mole_unimem_view_pool_size(void *handle, int *out);
int mole_unimem_virtual_offset(void *handle, int *out);
int mole_unimem_slot_ptr(void *handle, int p_id, int slot, void **out);
int mole_unimem_prefetch(void *handle, int layer, const void *const host_src[4], int base, int n);
int mole_unimem_prefetch_ids(void *handle, int layer, const void *const host_src[4], const int32_t *expert_ids,
                             int n, uint64_t tag);
/* The bookkeeping half of prefetch alone (_UniMem::prefetch, MOLE/cpp/umemory.cpp:131-154, exported by the
 * reference as pool_prefetch, MOLE/cpp/core.cpp:1425): reserve n slots for `layer` and return their addresses;
 * the caller fills them and orders its copies against the compute stream itself. */
int mole_unimem_reserve(void *handle, int layer, int n, void **slot_ptrs_out /* [4] */);
int mole_unimem_fetch_top(void *handle, int layer, int *n_out);
int mole_unimem_fetch(void *handle, const void *const host_src[4], int view_base, int base, int n,
                      int prefetched, void **slot_ptrs_out /* [4] */);
int mole_unimem_fetch_ids(void *handle, const void *const host_src[4], int view_base, const int32_t *expert_ids,
                          int n, int prefetched, uint64_t tag, void **slot_ptrs_out /* [4] */);
int mole_unimem_wait_params(void *handle, mole_stream_t compute_stream);
int mole_unimem_wait_slots(void *handle, int view_base, int n, mole_stream_t compute_stream);
int mole_unimem_release(void *handle, int view_base, int n, mole_stream_t compute_stream);
int mole_unimem_sync_tran(void *handle);
int mole_unimem_tran_stream(void *handle, mole_stream_t *out);
/* bytes moved host->device and the copy stream's busy time (events on the copy stream), summed over the copies
 * that mole_unimem_sync_tran() calls have waited for since the previous mole_unimem_copy_stats(); reading
 * resets the sums */
int mole_unimem_copy_stats(void *handle, uint64_t *bytes, float *busy_ms);
int mole_unimem_reuse_stats(void *handle, uint64_t *bytes);

/* Gradient write-back of offloaded experts; replaces _MOLECore::store_grad / _CPUParamCore::store_grad
 * (MOLE/cpp/core.cpp:77-103, MOLE/cpp/uparameter.cpp:68-83) and the "tranback" stream
 * (MOLE/cpp/stream.cpp:129-134).  dev_src[p] holds the gradients of n experts, [n, ...] contiguous, for
 * parameter kind p; they are copied to experts [base, base+n) of the pinned host arrays host_dst[p] on a
 * second library-owned stream once the work already enqueued on compute_stream has finished.  The caller
 * keeps dev_src alive until that stream has passed the copy (mole_unimem_tranback_stream tells which) and
 * reads the host arrays only after mole_unimem_sync_tranback().  Overwrites; accumulation is the caller's.
 * mole_unimem_writeback_stats: bytes and copy time of the write-backs that sync_tranback calls have waited for
 * since the previous read; reading resets the sums. */
int mole_unimem_store_grads(void *handle, void *const host_dst[4], const void *const dev_src[4], int base,
                            int n, mole_stream_t compute_stream);
/* The same for an explicit expert list: the i-th of the n experts in dev_src goes to host expert expert_ids[i].
 * mole_unimem_zero_grads_ids writes zeros to the listed host experts instead (the gradient of an expert that
 * received no rows), from a zeroed device slot the pool allocates on first use; it is ordered after the
 * write-backs already enqueued and waits for no compute. */
int mole_unimem_store_grads_ids(void *handle, void *const host_dst[4], const void *const dev_src[4],
                                const int32_t *expert_ids, int n, mole_stream_t compute_stream);
int mole_unimem_zero_grads_ids(void *handle, void *const host_dst[4], const int32_t *expert_ids, int n);
int mole_unimem_sync_tranback(void *handle);
int mole_unimem_tranback_stream(void *handle, mole_stream_t *out);
int mole_unimem_writeback_stats(void *handle, uint64_t *bytes, float *busy_ms);

/* Optimizer state of offloaded experts in the backward pipeline; replaces the moment fetches and the
 * parameter / moment stores of _MOLECore::instant_adam (MOLE/cpp/core.cpp:864-935:
 * fetch_batch_cpu_mome/vari/grad + _ParamProxy::fetch on the tran stream after comp_event,
 * store_batch_cpu_para/mome/vari on the tranback stream).
 * mole_unimem_load_state: count host->device copies of bytes[i] from pinned host_src[i] to dev_dst[i] on
 * the library's copy stream, which first waits for the work already enqueued on compute_stream (the
 * previous users of dev_dst) and, when after_writeback != 0, for the write-backs enqueued so far (set it when
 * host_src may be the target of one, e.g. gradients stored by the previous micro-step; it serialises the two
 * copy directions); compute_stream then waits for the copies.
 * mole_unimem_store_state: count device->host copies on the write-back stream once the work already
 * enqueued on compute_stream has finished; lifetime and synchronisation rules as for
 * mole_unimem_store_grads. */
int mole_unimem_load_state(void *handle, void *const dev_dst[], const void *const host_src[], const size_t bytes[],
                           int count, int after_writeback, mole_stream_t compute_stream);
int mole_unimem_store_state(void *handle, void *const host_dst[], const void *const dev_src[], const size_t bytes[],
                            int count, mole_stream_t compute_stream);

/* Fused Adam / AdamW step on a flat array of n elements; replaces _MOLECore::adam
 * (MOLE/cpp/define.hpp:543-579) as called four times per expert batch by instant_adam
 * (MOLE/cpp/core.cpp:917-920).  p, g: dtype (fp32 or bf16); m, v: fp32, updated in place; p_out: dtype, may
 * be p itself or a separate buffer (the reference's write-back variant keeps p and returns p_back).
 * t is the step count already incremented (the reference uses its stored counter + 1); lam is the weight
 * decay: adamw != 0 scales p by (1 - lam lr) first, otherwise g += lam p.  In the reference's order:
 * m = b1 m + (1-b1) g;  v = b2 v + (1-b2) g g;  p_out = p - lr (m / (1-b1^t)) / (sqrt(v / (1-b2^t)) + eps).
 * All pointers 16-byte aligned. */
int mole_adam_step(const void *p, const void *g, float *m, float *v, void *p_out, size_t n, int dtype,
                   float beta1, float beta2, int t, float lr, float lam, float eps, int adamw,
                   mole_stream_t stream);

/* acc[i] += add[i] over n elements of dtype, rounded once per element: the sum of a micro-step's gradients and the
 * running sum fetched from the host; replaces the host-side addition of grad_accumulate
 * (MOLE/cpp/data_transfer.cpp:9-12, called from store_grad, MOLE/cpp/core.cpp:77-103).  16-byte aligned. */
int mole_grad_add(void *acc, const void *add, size_t n, int dtype, mole_stream_t stream);

/* Greedy cross-layer prefetch assignment; replaces fast_assign_prefetch
 * (MOLE/cpp/core.cpp:1302-1345).  lp_out [n]; gp_out holds up to gp_cap triples
 * (from_layer, for_layer, count), *gp_n the number written. */
int mole_fast_assign_prefetch(int P, const int *Fv, const int *Ev, int n, int *lp_out, int *gp_out,
                              int gp_cap, int *gp_n);

#ifdef __cplusplus
}
#endif
#endif /* MOLE_HIP_H */
