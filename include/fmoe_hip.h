/*
 * fmoe_hip.h -- C ABI of the MI355X (gfx950) single-GPU MoE-layer hot path.
 *
 * Every entry point is `extern "C"`, takes plain device pointers, sizes and a
 * HIP stream (as void*), launches asynchronously on that stream and returns 0
 * or a negative fmoe_status.  Nothing here exits the process; the text of the
 * last failure on the calling thread is available from fmoe_last_error().
 *
 * Citations name the interface of the reference (laekov/fastmoe) that each
 * entry point stands in for, as path:line in the reference tree.
 *
 * Conventions
 *   gate / pos      int64, as produced by torch.topk and consumed by the
 *                   reference's Python (fmoe/functions.py:28-49).
 *   counts          int32 for histograms and capacities (cuda/balancing.cu:6-8),
 *                   int64 where the reference hands them to Python.
 *   slots           the N = tokens * top_k routed entries of `gate`, flat index
 *                   i = token * top_k + j.
 *   rows            the N_valid slots that survived (gate != -1), grouped by
 *                   expert; row r of a dispatch buffer holds slot pos[r].
 *   seg_off         int32[E+1] exclusive prefix of per-expert row counts;
 *                   expert e owns rows [seg_off[e], seg_off[e+1]).
 *   inv             int32[N]: inv[pos[r]] = r, and -1 for dropped slots.
 *   order           rows of one expert are in ascending slot index (stable),
 *                   which is one legal outcome of the reference's atomics.
 */
#ifndef FMOE_HIP_H_
#define FMOE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum fmoe_status {
  FMOE_OK = 0,
  FMOE_ERR_INVALID = -1,     /* bad argument (null pointer, negative size, ...) */
  FMOE_ERR_UNSUPPORTED = -2, /* shape / dtype outside what the kernels handle   */
  FMOE_ERR_HIP = -3,         /* a HIP runtime call or a launch failed           */
  FMOE_ERR_WORKSPACE = -4    /* workspace missing or too small                  */
} fmoe_status;

typedef enum fmoe_dtype {
  FMOE_F32 = 0,
  FMOE_F64 = 1,
  FMOE_F16 = 2,
  FMOE_BF16 = 3
} fmoe_dtype;

/* Largest number of experts the routing kernels keep in LDS. */
#define FMOE_MAX_EXPERTS 4096
/* Largest top_k of the fused gate kernels. */
#define FMOE_MAX_GATE_TOP_K 16

/* Library identification and error text (thread-local, never NULL). */
const char* fmoe_version(void);
const char* fmoe_last_error(void);

/*
 * Optional one-time set-up of the CURRENT GPU, on `stream` (waited for before the
 * call returns): everything the entry points below otherwise do lazily at their
 * first call on a GPU, namely the activation tables of the 16-bit kernels and the
 * device address of fmoe_route_static's built-in buffer.  Callers that capture HIP
 * graphs call it once per GPU before the first capture; everybody else may skip it.
 * Thread-safe and idempotent.  No counterpart in the reference (its extension has
 * no set-up of its own beyond the stream manager, cuda/stream_manager.cpp:75-93).
 */
int fmoe_init(void* stream);

/* ------------------------------------------------------------------ routing */

/*
 * Histogram of gate indices: expert_count[e] += #{i : gate_idx[i] == e}.
 * Entries equal to -1 or outside [0, n_expert) are skipped; the output is
 * accumulated into, not overwritten (the caller zero-fills).
 * Replaces fmoe_cuda.expert_count: cuda/fmoe_cuda.cpp:43-45,
 * cuda/local_exchange.cu:22-32, kernel cuda/local_exchange.cuh:36-78.
 */
int fmoe_expert_count(const int64_t* gate_idx, int64_t numel,
                      int32_t* expert_count, int32_t n_expert, void* stream);

/*
 * Bytes of device workspace needed by fmoe_assign_pos, fmoe_route and
 * fmoe_prune_gate_by_capacity for `numel` slots and `n_expert` experts.
 * Returns a negative fmoe_status on bad arguments.
 */
int64_t fmoe_route_workspace_bytes(int64_t numel, int32_t n_expert);

/*
 * Positions from an inclusive cumulative count.
 * In:  cum_count[e] = sum_{e'<=e} count[e'] (int32), gate (int64, numel slots).
 * Out: pos[off[e] .. cum_count[e]) = the slots routed to e in ascending slot
 *      index, off[e] = cum_count[e] - count[e].  On return cum_count[e] = off[e],
 *      the state the reference's atomicSub leaves behind.
 * Replaces fmoe_cuda.assign_pos: cuda/fmoe_cuda.cpp:39-42,
 * cuda/local_exchange.cu:5-20, kernel cuda/local_exchange.cuh:5-26.
 */
int fmoe_assign_pos(int32_t* cum_count, const int64_t* gate, int64_t* pos,
                    int64_t numel, int32_t n_expert, void* workspace,
                    int64_t workspace_bytes, void* stream);

/*
 * Fused routing metadata, no host synchronisation:
 *   count64[e]  (optional, int64[E])   rows per expert, overwritten
 *   seg_off     (int32[E+1])           exclusive prefix, seg_off[E] = N_valid
 *   pos         (int64[numel])         first N_valid entries written
 *   inv         (optional, int32[numel])
 * Stands in for fmoe.functions.count_by_gate + prepare_forward
 * (fmoe/functions.py:28-75) without their five device-to-host copies.
 * Three launches (histogram, scans, placement); up to 4096 slots and 512
 * experts one workgroup does all three in a single launch, same results.  The
 * workspace is required either way.
 */
int fmoe_route(const int64_t* gate, int64_t numel, int32_t n_expert,
               int64_t* count64, int32_t* seg_off, int64_t* pos, int32_t* inv,
               void* workspace, int64_t workspace_bytes, void* stream);

/*
 * fmoe_route for callers that cannot allocate: the three-launch kernels and
 * the same results, with the per-block histograms in a buffer built into the library
 * (FMOE_ROUTE_STATIC_SCRATCH_BYTES per GPU, held until the process ends) instead
 * of a workspace argument.  It calls no allocating routine, so it may be used
 * under HIP graph capture (after fmoe_init(), or one eager call, on that GPU: the
 * first use on a GPU asks the runtime for the buffer's address), in serving loops
 * and in harnesses that forbid hipMalloc.  Sizes whose workspace (fmoe_route_workspace_bytes) exceeds the
 * buffer are rejected with FMOE_ERR_WORKSPACE.  All calls on one GPU share the
 * buffer: calls that overlap in time on one GPU (two streams) race.
 * No counterpart in the reference; it exists for the callers named above.
 */
#define FMOE_ROUTE_STATIC_SCRATCH_BYTES (4 * 1024 * 1024)
int fmoe_route_static(const int64_t* gate, int64_t numel, int32_t n_expert,
                      int64_t* count64, int32_t* seg_off, int64_t* pos, int32_t* inv,
                      void* stream);

/* ----------------------------------------------------------------- capacity */

/*
 * eca[w*E+e] = share of expert e's capacity granted to worker w, workers
 * served in ascending w: grant = proposal if remaining >= proposal, remaining
 * if remaining >= 0, else 0; remaining -= proposal (the full proposal, also
 * when clipped).  cap[e] is left holding `remaining`, as the reference's
 * atomicSub leaves it.  Proposals are truncated to int32 as in the reference.
 * Replaces fmoe_cuda.limit_by_capacity: cuda/fmoe_cuda.cpp:63-65,
 * cuda/balancing.cu:9-22, kernel cuda/balancing.cuh:5-30.
 */
int fmoe_limit_by_capacity(const int64_t* ec, int32_t* cap, int64_t* eca,
                           int64_t n_expert, int64_t n_worker, void* stream);

/*
 * new_gate_idx[i] = gate_idx[i] if fewer than ec[gate_idx[i]] earlier slots
 * (ascending i) chose the same expert, else -1.  Entries outside [0, E*W)
 * (including -1) are copied through.  ec[e] is left at ec[e] - count[e], the
 * state the reference's atomicSub leaves behind.
 * Replaces fmoe_cuda.prune_gate_by_capacity: cuda/fmoe_cuda.cpp:66-68,
 * cuda/balancing.cu:24-39, kernel cuda/balancing.cuh:32-56.
 */
int fmoe_prune_gate_by_capacity(const int64_t* gate_idx, int64_t* new_gate_idx,
                                int32_t* ec, int64_t numel, int64_t n_expert,
                                int64_t n_worker, void* workspace,
                                int64_t workspace_bytes, void* stream);

/* ----------------------------------------------------------------- dispatch */

/*
 * out[r] = inp[idx[r] / idx_div] for r < n_rows (rows of `d` elements).
 * If n_rows_dev is not NULL it points at a device int32 holding the live row
 * count (<= n_rows) and rows beyond it are left untouched.
 * Replaces fmoe.functions._local_scatter (fmoe/functions.py:78-80) and the
 * `pos // top_k` that precedes it (fmoe/layers.py:49-53).
 */
int fmoe_local_scatter(const void* inp, const int64_t* idx, void* out,
                       int64_t n_rows, int64_t d, int64_t idx_div,
                       const int32_t* n_rows_dev, int dtype, void* stream);

/*
 * out[inv[t * top_k + j]] = inp[t] for every slot with inv >= 0: the same rows
 * as fmoe_local_scatter(inp, pos, ..., idx_div = top_k) writes, produced in
 * token order from the inverse map of fmoe_route (a token row is read once for
 * its top_k copies).  inp [n_tokens, d], out [>= live rows, d]; top_k <= 64.
 * Replaces fmoe.functions._local_scatter (fmoe/functions.py:78-80) in
 * MOEScatter.forward (functions.py:100-121) when the inverse map is at hand.
 */
int fmoe_scatter_tokens(const void* inp, const int32_t* inv, void* out,
                        int64_t n_tokens, int64_t top_k, int64_t d, int dtype,
                        void* stream);

/*
 * overlap == 0: out = 0 [out_rows, d]; out[pos[r]] = inp[r]  (pos distinct).
 * overlap != 0: out[p] = sum over {r : pos[r] == p} inp[r]; f32/f64 only
 *               (device float atomics, summation order unspecified, as with
 *               the reference's index_add_).
 * Replaces fmoe.functions._local_gather (fmoe/functions.py:83-90).
 */
int fmoe_local_gather(const void* inp, const int64_t* pos, void* out,
                      int64_t n_rows, int64_t out_rows, int64_t d,
                      const int32_t* n_rows_dev, int overlap, int dtype,
                      void* stream);

/*
 * Gather fused with the top-k weighted combine:
 *   y[t] = sum_j score[t*k+j] * buf[inv[t*k+j]]   (dropped slots add 0)
 * fp32 accumulation (fp64 for FMOE_F64), one rounding.
 * Replaces MOEGather.forward + torch.bmm (fmoe/functions.py:150-176,
 * fmoe/layers.py:281-295).
 */
int fmoe_gather_combine_fwd(const void* buf, const int32_t* inv,
                            const void* score, void* y, int64_t n_tokens,
                            int64_t top_k, int64_t d, int dtype, void* stream);

/*
 * Backward of fmoe_gather_combine_fwd, written straight into expert order:
 *   dbuf[inv[i]] = score[i] * dy[i / k]          (live slots)
 *   dscore[i]    = <dy[i / k], buf[inv[i]]>      (0 for dropped slots)
 * Replaces the bmm backward + MOEGather.backward (fmoe/functions.py:178-193).
 */
int fmoe_gather_combine_bwd(const void* dy, const void* buf, const int32_t* inv,
                            const void* score, void* dbuf, void* dscore,
                            int64_t n_tokens, int64_t top_k, int64_t d,
                            int dtype, void* stream);

/*
 * Backward of the scatter: dx[t] = sum_j dbuf[inv[t*k+j]] over live slots, in
 * ascending j with fp32 accumulation (deterministic; no float atomics).
 * Replaces MOEScatter.backward (fmoe/functions.py:126-142).
 */
int fmoe_scatter_reduce(const void* dbuf, const int32_t* inv, void* dx,
                        int64_t n_tokens, int64_t top_k, int64_t d, int dtype,
                        void* stream);

/* ------------------------------------------------------------ expert GEMMs */

/*
 * Y[seg_e] = X[seg_e] * W_e^T (+ b_e) for every expert in one launch.
 *   x [n_rows, in_feat], w [E, out_feat, in_feat], bias [E, out_feat] or NULL,
 *   y [n_rows, out_feat]; seg_off is a DEVICE int32[E+1].
 * Rows at or beyond seg_off[E] are not written.  Empty experts cost nothing.
 * bf16/f16: MFMA with fp32 accumulation.  f32/f64: accumulation in the same
 * type, on the matrix cores when both feature sizes are multiples of 4, else in
 * a scalar kernel.
 * Replaces fmoe_cuda.linear_forward: cuda/fmoe_cuda.cpp:48-53,
 * cuda/parallel_linear.cu:5-50, cuda/parallel_linear.cuh:55-89.
 */
int fmoe_grouped_linear_fwd(const void* x, const void* w, const void* bias,
                            const int32_t* seg_off, void* y, int64_t n_rows,
                            int64_t in_feat, int64_t out_feat,
                            int64_t n_expert, int dtype, void* stream);

/*
 * dX[seg_e] = dY[seg_e] * W_e;  dW_e = dY[seg_e]^T * X[seg_e];
 * db_e = column sums of dY[seg_e] (only if dbias != NULL).
 * Experts without rows get dW_e = 0 and db_e = 0.  Any of dx, dw, dbias may
 * be NULL to skip that product.
 * Replaces fmoe_cuda.linear_backward: cuda/fmoe_cuda.cpp:54-60,
 * cuda/parallel_linear.cu:53-96, cuda/parallel_linear.cuh:91-163 and the
 * column_reduce kernel cuda/parallel_linear.cuh:8-53.
 */
int fmoe_grouped_linear_bwd(const void* dy, const void* x, const void* w,
                            const int32_t* seg_off, void* dx, void* dw,
                            void* dbias, int64_t n_rows, int64_t in_feat,
                            int64_t out_feat, int64_t n_expert, int dtype,
                            void* stream);

/*
 * Forward of the first layer of the reference's expert with its activation
 * (fmoe/transformer.py:25-33: htoh4 -> activation): y as fmoe_grouped_linear_fwd
 * writes it (the pre-activations, which the backward needs) and y_act = gelu(y),
 * the exact GELU of torch.nn.GELU().  Where the bf16 matrix-core kernel runs, both
 * leave the same output tiles (the activation kernel's own table of gelu(x) for
 * 16-bit x, applied to the rounded y: the same bits as fmoe_gelu_fwd over y); for
 * other dtypes and shapes, and below about 768 rows per expert (where the separate
 * kernel is as fast), the entry point runs that kernel behind the GEMM
 * (fmoe_set_gemm_path(6) makes it do so always).  Rows of y_act behind
 * seg_off[n_expert] are left untouched, like those of y.
 */
int fmoe_grouped_linear_fwd_act(const void* x, const void* w, const void* bias,
                                const int32_t* seg_off, void* y, void* y_act,
                                int64_t n_rows, int64_t in_feat, int64_t out_feat,
                                int64_t n_expert, int dtype, void* stream);

/*
 * fmoe_grouped_linear_bwd for a layer whose input is act = gelu(act_pre), with
 * the activation's backward folded in: dx = (dY[seg_e] * W_e) .* gelu'(act_pre),
 * x being act (dW is unchanged).  act_pre is [n_rows, in_feat].  bf16 on the
 * matrix-core kernel applies the factor in the tile epilogue, so the product
 * dY * W never reaches memory; every other case runs fmoe_gelu_bwd over dx, with
 * the same bits out.  The first bf16 call builds the activation tables (see
 * fmoe_gelu_fwd).
 * Replaces, for the second linear layer of an expert, fmoe_cuda.linear_backward
 * followed by the backward of the activation in between
 * (fmoe/transformer.py:25-33: htoh4 -> activation -> h4toh).
 */
int fmoe_grouped_linear_bwd_act(const void* dy, const void* x, const void* w,
                                const int32_t* seg_off, const void* act_pre,
                                void* dx, void* dw, void* dbias, int64_t n_rows,
                                int64_t in_feat, int64_t out_feat,
                                int64_t n_expert, int dtype, void* stream);

/*
 * The grouped linear layer for experts whose parameters are SEPARATE allocations:
 * the reference's FMoETransformerMLP keeps one single-expert module per expert
 * (fmoe/transformer.py:51-55), and its GEMM loop addresses every expert's weight
 * through a pointer of its own (cuda/parallel_linear.cuh:69-87).  w_ptrs and
 * bias_ptrs (may be NULL) are DEVICE arrays of n_expert device pointers: expert e's
 * weight [out_feat, in_feat] is at w_ptrs[e], its bias [out_feat] at bias_ptrs[e];
 * every pointer 16-byte aligned.  Everything else is as in the entry points above:
 *   _fwd_ptrs  = fmoe_grouped_linear_fwd, or with y_act != NULL
 *                fmoe_grouped_linear_fwd_act;
 *   _bwd_ptrs  = fmoe_grouped_linear_bwd, or with act_pre != NULL
 *                fmoe_grouped_linear_bwd_act.  dw and dbias stay single [E, out, in]
 *                and [E, out] arrays (the caller hands out per-expert views of them).
 * No weight is copied, and the results carry the same bits as a call on the
 * concatenated weights.
 */
int fmoe_grouped_linear_fwd_ptrs(const void* x, const void* const* w_ptrs,
                                 const void* const* bias_ptrs, const int32_t* seg_off,
                                 void* y, void* y_act, int64_t n_rows, int64_t in_feat,
                                 int64_t out_feat, int64_t n_expert, int dtype,
                                 void* stream);
int fmoe_grouped_linear_bwd_ptrs(const void* dy, const void* x, const void* const* w_ptrs,
                                 const int32_t* seg_off, const void* act_pre, void* dx,
                                 void* dw, void* dbias, int64_t n_rows, int64_t in_feat,
                                 int64_t out_feat, int64_t n_expert, int dtype,
                                 void* stream);

/*
 * table[i] = host_ptrs[i] for i < n: fills a DEVICE array of pointers (the w_ptrs /
 * bias_ptrs above) from a HOST array, asynchronously on `stream`; the values travel
 * as kernel arguments, so the host array may be reused as soon as the call returns
 * and nothing is synchronised.  The counterpart of the host-side pointer arithmetic
 * of cuda/parallel_linear.cuh:69-87.
 */
int fmoe_pointer_table(const void* const* host_ptrs, int64_t n, const void** table,
                       void* stream);

/*
 * seg_off (device int32[E+1]) from HOST int64 counts, the form in which the
 * reference passes counts to its linear ops (cuda/parallel_linear.cuh:69-70
 * dereferences expert_count on the host).  `seg_off` must stay alive until
 * the stream reaches the copy.
 */
int fmoe_seg_off_from_host_counts(const int64_t* expert_count_host,
                                  int64_t n_expert, int32_t* seg_off,
                                  void* stream);

/*
 * Top-k gate in one pass: for every token the top_k largest of its n_expert
 * logits (row-major logits[n_tokens][n_expert]) and the softmax over those
 * top_k values:
 *   idx[t][j]   = expert of the j-th largest logit (equal logits: lower index first)
 *   score[t][j] = exp(v_j - v_0) / sum_i exp(v_i - v_0)      (dtype of the logits)
 * Replaces torch.topk + F.softmax of fmoe/gates/naive_gate.py:31-38; torch.topk
 * leaves the order of its results open, this call returns them by descending
 * logit.  top_k <= min(n_expert, FMOE_MAX_GATE_TOP_K).  A NaN logit ranks above
 * every number, as in torch.topk, so a token with NaN logits gets NaN scores.
 */
int fmoe_topk_softmax_fwd(const void* logits, int64_t n_tokens, int32_t n_expert,
                          int32_t top_k, int64_t* idx, void* score, int dtype,
                          void* stream);

/*
 * Backward of fmoe_topk_softmax_fwd with respect to the logits:
 *   dlogits[t][idx[t][j]] = score_j * (dscore_j - sum_i dscore_i * score_i)
 * and zero for every other expert (all n_tokens * n_expert entries are written).
 * Replaces the autograd chain of naive_gate.py:31-38 (softmax backward, zero
 * fill, scatter of the top-k gradient).
 */
int fmoe_topk_softmax_bwd(const void* dscore, const void* score, const int64_t* idx,
                          void* dlogits, int64_t n_tokens, int32_t n_expert,
                          int32_t top_k, int dtype, void* stream);

/*
 * y[i] = gelu(x[i]) = 0.5 x (1 + erf(x / sqrt 2)) over n elements, and
 * dx[i] = dy[i] * gelu'(x[i]): the activation between the two expert layers,
 * fmoe/transformer.py:28-30 with the default torch.nn.GELU() of
 * transformer.py:45 (the reference calls the torch module; these kernels take
 * its place on the GPU).  bf16/f16 read gelu(x) (computed in double precision,
 * rounded once) and gelu'(-|x|) (f32) from tables held in LDS; f32/f64 evaluate
 * erf.  Inputs and outputs must not overlap.  n_rows_dev (DEVICE int32, may be
 * NULL) with row_len tells that only the first *n_rows_dev rows of row_len
 * elements are live, as in the expert-ordered buffers behind a capacity limit:
 * the rest is neither read nor written.  The first 16-bit call on a GPU builds
 * that GPU's tables on `stream` and waits for them (thread-safe); that one call
 * cannot be captured into a HIP graph and returns FMOE_ERR_UNSUPPORTED there.
 */
int fmoe_gelu_fwd(const void* x, void* y, int64_t n, const int32_t* n_rows_dev,
                  int64_t row_len, int dtype, void* stream);
int fmoe_gelu_bwd(const void* dy, const void* x, void* dx, int64_t n,
                  const int32_t* n_rows_dev, int64_t row_len, int dtype, void* stream);

/*
 * Selects the grouped-GEMM kernel family for the CALLING THREAD's later calls:
 * 0 = automatic (MFMA where the shape allows, tile shape from the library's cost
 * model), 1 = force the scalar kernel, 2..5 = MFMA with bf16/f16 tile
 * configuration 1..4 forced (256x256, 128x256, 128x128, 256x256 with K slices of
 * 64; f32/f64 have one tile shape), 6 = automatic, with the forward activation of
 * fmoe_grouped_linear_fwd_act always as a kernel of its own.  A testing aid with
 * no counterpart in the reference; the setting is thread-local (every thread
 * starts at 0), so concurrent callers do not disturb each other.
 */
int fmoe_set_gemm_path(int path);

#ifdef __cplusplus
}
#endif
#endif /* FMOE_HIP_H_ */
