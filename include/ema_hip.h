/*
 * ema_hip.h -- C ABI of libema_hip.so: the EMA chunked scan (forward and backward) as
 * hand-written HIP kernels for gfx950 (MI355X).
 *
 * Every entry point replaces one launcher of the reference repository
 * kartiksrinivas007/triton-kernels (a Python function that allocates its output and starts
 * one Triton kernel); the citation on each declaration is that launcher, with paths
 * relative to the reference root.
 *
 * Conventions
 *   - All pointers are DEVICE pointers.  The caller allocates every input, output and
 *     workspace; the library never allocates, frees or keeps a pointer.
 *   - Work is only enqueued on `stream` (a hipStream_t passed as void*; NULL = the null
 *     stream).  No entry point synchronises or reads anything back, so all of them may be
 *     captured into a HIP graph.
 *   - Sequence tensors (x, y, dy, dx) are addressed as
 *         ptr[b * s_b + l * s_l + h * s_h + t],   b < batch, l < seqlen, h < nheads, t < dim
 *     with strides in ELEMENTS and a unit stride along `dim`.  The reference's flat
 *     layout (B, L, T) is nheads = 1; the headed layout (b, L, nh, d) is s_b = L*nh*d,
 *     s_l = nh*d, s_h = d.  The log-decay A (float32) is addressed the same way without
 *     the `dim` axis.  A sequence index n = b * nheads + h numbers the independent scans;
 *     N = batch * nheads.
 *   - Chunked intermediates are dense float32: cs (N, C, Q), states / prev / ds / g
 *     (N, C, T), final (N, T), per-chunk scalars (N, C); C = ceil(seqlen / chunk).
 *   - `dtype` is the element type of the sequence tensors (ema_dtype); accumulation is
 *     always float32.  dim must be a multiple of 8 (bf16) or 4 (f32) and row starts must
 *     be 16-byte aligned.
 *   - Return value: EMA_OK (0) or a negative ema_status.  Arguments are validated before
 *     anything is launched; nothing is thrown across the boundary.
 *   - Workspaces of the single-pass entry points (ema_fwd, ema_bwd, ema_seq_fwd, ema_seq_bwd)
 *     begin with an ema_chain_header followed by the words through which the tiles of the
 *     chained scan hand their state to each other (the chained part); per-call scratch follows.
 *     Every word of the chained part is tagged with the epoch of the call that wrote it, so
 *     nothing has to be cleared between calls: a buffer that was zero-filled once
 *     (ema_workspace_clear, or any memset) serves any number of calls of these four entry points
 *     on one problem shape (batch * nheads, seqlen, dim), forward and backward alike, one after
 *     the other.  Pass workspace_ready = 1 for such a buffer and the call launches no clearing
 *     kernel; with workspace_ready = 0 the call first clears the chained part (one more small
 *     launch), which is right for a buffer of unknown contents.  A ready buffer must have held
 *     nothing but this library's words since it was cleared (the tags are compared as plain
 *     words); ema_seq_fwd, whose workspace is the chained part alone, may change shape from
 *     call to call on one buffer.  Calls that share a workspace must not overlap in time.  A
 *     buffer must be cleared again after 2^30 calls, and after a call that was aborted or that
 *     the header's error word reports.
 */
#ifndef EMA_HIP_H
#define EMA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  EMA_OK = 0,
  EMA_ERR_NULL = -1,        /* a required pointer is NULL */
  EMA_ERR_SHAPE = -2,       /* a dimension is <= 0 or out of the supported range */
  EMA_ERR_ALIGN = -3,       /* dim / strides / pointers break the 16-byte rule */
  EMA_ERR_DTYPE = -4,       /* unknown ema_dtype */
  EMA_ERR_UNSUPPORTED = -5, /* a feature the reference also rejects */
  EMA_ERR_LAUNCH = -6,      /* hipGetLastError() after a launch was not hipSuccess */
  EMA_ERR_TOO_LARGE = -7    /* the problem needs more than the fixed scratch of ema_seq_fwd_static */
} ema_status;

typedef enum { EMA_F32 = 0, EMA_BF16 = 1 } ema_dtype;

/* How the per-position coefficient of the sequence-level entry points is given. */
typedef enum {
  EMA_FORM_LOG_DECAY = 0,  /* A:  y[t] = exp(min(A[t], 0)) * y[t-1] + x[t]           */
  EMA_FORM_PROBABILITY = 1 /* p:  y[t] = (1 - p[t]) * y[t-1] + p[t] * x[t]           */
} ema_form;

/* What a workspace of the single-pass entry points begins with (256 bytes, device memory).  The
 * library maintains it; a caller may read `error` (for instance together with the results) and
 * may set `spin_limit` between calls.
 *   error      non-zero once a tile's bounded wait for its predecessor has run out in some call
 *              since the buffer was last cleared (a predecessor that never published: a
 *              workspace that was not ready, overlapping calls on one workspace, or a device so
 *              oversubscribed that resident workgroups stopped making progress).  The affected
 *              outputs are NaN; the call itself still returns EMA_OK, since nothing is read back.
 *   spin_limit polls of one word before a wait gives up; 0 = the built-in 2^20. */
typedef struct {
  uint32_t ticket;     /* next tile to hand out; zero between calls */
  uint32_t done;       /* workgroups that have left the running call; zero between calls */
  uint32_t epoch;      /* epoch of the last completed call */
  uint32_t error;
  uint32_t spin_limit;
  uint32_t reserved[59];
} ema_chain_header;

/* Zero-fills `bytes` bytes of device memory at `workspace` (16-byte aligned) with a kernel on
 * `stream`: the state in which workspace_ready = 1 may be passed. */
int ema_workspace_clear(void* workspace, size_t bytes, void* stream);

/* Measurement aid (no counterpart in the reference): dst = a, or dst = a ^ b when b is not NULL,
 * `bytes` bytes (a multiple of 16; pointers 16-byte aligned), one 16-byte piece per thread with
 * non-temporal accesses.  bench.py times it back to back over rotating buffers: what the plainest
 * streaming kernel sustains on the device is the practical ceiling next to which the scan
 * kernels' rates are reported. */
int ema_stream_copy(const void* a, const void* b, void* dst, size_t bytes, void* stream);

/* Measurement aid (no counterpart in the reference): copies a (slabs, rows, row_bytes) byte tensor
 * (rows a multiple of 128, row_bytes a multiple of 512) in the access pattern of the single-pass
 * kernels: one persistent workgroup per compute unit, tiles of 128 rows x 512 bytes in chunk-major
 * order, 8 bytes per lane and row.  rowmap 0: sixteen waves with 8 consecutive rows each, the shape
 * in which the two kernels load and store; rowmap 3: eight waves with 16 consecutive rows each;
 * rowmap 1: eight waves, the rows of a wave 8 apart and slabs rotated against each other, which is
 * the order the memory system sustains the highest rate for; rowmap 2: memory is touched as with
 * rowmap 1 and every wave still gets 16 consecutive rows into its registers, the rows changing
 * hands through LDS on the way in and on the way out.  Other values: EMA_ERR_UNSUPPORTED.  src2 (may
 * be NULL; rowmap 0 only): a second input of the same layout, dst = src ^ src2, the backward kernel's
 * two inputs and one output.  bench.py reports all of them next to the plain streaming copy: rowmap 0
 * is the ceiling of the scan kernels' own pattern. */
int ema_tile_pattern_copy(const void* src, const void* src2, void* dst, int64_t slabs, int64_t rows,
                          int64_t row_bytes, int rowmap, void* stream);

/* Largest chunk size accepted by every entry point. */
#define EMA_MAX_CHUNK 1024

const char* ema_version(void);
const char* ema_status_string(int status);

/* ---------------------------------------------------------------- forward stages ---- */

/* F1: cs[n,c,q] = sum_{j<=q} A[n, c*Q+j], restarting every chunk, positions past seqlen
 * adding 0.  Replaces ema_chunk_cumsum_fwd, kernels/ema_kernels/ema_cumsum.py:66-80. */
int ema_chunk_cumsum_fwd(const float* A, int64_t a_sb, int64_t a_sl, int64_t a_sh,
                         float* cs, int64_t batch, int64_t nheads, int64_t seqlen,
                         int64_t chunk, void* stream);

/* F2: states[n,c,t] = sum_q exp(min(cs[n,c,Q-1]-cs[n,c,q],0)) * x[n,c*Q+q,t].
 * Replaces _ema_chunk_state_fwd, kernels/ema_kernels/ema_state_fwd.py:130-163. */
int ema_chunk_state_fwd(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype,
                        const float* cs, float* states, int64_t batch, int64_t nheads,
                        int64_t seqlen, int64_t dim, int64_t chunk, void* stream);

/* F3: S_0 = 0; prev[n,c] = S_c; S_{c+1} = exp(cs_last[n,c]) * S_c + states[n,c];
 * final[n] = S_C.  cs_last is addressed as cs_last[n*cl_sn + c*cl_sc] so that the strided
 * view cs[..., -1] can be passed without a copy.
 * Replaces _ema_state_passing_fwd, kernels/ema_kernels/ema_state_pass.py:125-154. */
int ema_state_passing_fwd(const float* states, const float* cs_last, int64_t cl_sn,
                          int64_t cl_sc, float* prev, float* final_state, int64_t nseq,
                          int64_t nchunks, int64_t dim, void* stream);

/* F4: y[n,c*Q+m,t] = exp(min(cs[m],0)) * prev[n,c,t]
 *                   + sum_{k<=m} exp(min(cs[m]-cs[k],0)) * x[n,c*Q+k,t].
 * Replaces _ema_scan_fwd, kernels/ema_kernels/ema_scan_fwd.py:161-193. */
int ema_scan_fwd(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype,
                 const float* cs, const float* prev, void* y, int64_t y_sb, int64_t y_sl,
                 int64_t y_sh, int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim,
                 int64_t chunk, void* stream);

/* Bytes of workspace ema_fwd needs. */
size_t ema_fwd_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim,
                               int64_t chunk);

/* Whole forward.  Outputs y, cs (N,C,Q), prev (N,C,T) (state entering each chunk) and
 * final (N,T).  When chunk is a multiple of 128 x is read ONCE: the scan runs on 128-row
 * chunks and the inter-chunk state is handed from tile to tile inside the kernel (chained
 * scan with look-back) instead of by separate F2 / F3 passes; prev128, if not NULL,
 * receives the states entering each 128-row chunk, (N, ceil(seqlen/128), T), which
 * ema_bwd accepts to skip their recomputation.  For other chunk sizes F1..F4 run in
 * sequence and prev128 must be NULL.  ev_start / ev_stop (hipEvent_t, may be NULL) are
 * recorded on the stream right before and after the kernel(s) that read x, so that a
 * caller can time them apart from the small kernel that writes cs.  workspace_ready: see the
 * conventions above (ignored when chunk is not a multiple of 128).
 * Replaces _ema_matmul_scan_combined_fwd, kernels/ema_kernels/ema_combined_fwd.py:12-45. */
int ema_fwd(const float* A, int64_t a_sb, int64_t a_sl, int64_t a_sh, const void* x,
            int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, void* y, int64_t y_sb,
            int64_t y_sl, int64_t y_sh, float* cs, float* prev, float* final_state,
            float* prev128, void* workspace, size_t workspace_bytes, int workspace_ready,
            int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim, int64_t chunk, void* stream,
            void* ev_start, void* ev_stop);

/* --------------------------------------------------------------- backward stages ---- */

/* B1: ds[n,c,t] = sum_m exp(cs[n,c,m]) * dy[n,c*Q+m,t].
 * Replaces _ema_chunk_scan_bwd_dstates, kernels/ema_kernels_bwd/ema_scan_bwd.py:132-153. */
int ema_chunk_scan_bwd_dstates(const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh,
                               int dtype, const float* cs, float* ds, int64_t batch,
                               int64_t nheads, int64_t seqlen, int64_t dim, int64_t chunk,
                               void* stream);

/* Bytes of workspace ema_state_passing_bwd needs (per-wave partial dot products). */
size_t ema_state_passing_bwd_workspace_bytes(int64_t nseq, int64_t nchunks, int64_t dim);

/* B2: g[n,C-1] = 0; g[n,c-1] = exp(cs_last[n,c]) * g[n,c] + ds[n,c];
 * ddA_chunk[n,c] = exp(cs_last[n,c]) * <prev[n,c], g[n,c]>, ddA_chunk[n,0] = 0.
 * Replaces _ema_state_passing_bwd,
 * kernels/ema_kernels_bwd/ema_state_passing_bwd_dstates.py:103-183. */
int ema_state_passing_bwd(const float* prev, const float* cs_last, int64_t cl_sn,
                          int64_t cl_sc, const float* ds, float* g, float* ddA_chunk,
                          void* workspace, size_t workspace_bytes, int64_t nseq,
                          int64_t nchunks, int64_t dim, void* stream);

/* B3: dx[n,c*Q+m,t] = exp(min(cs[Q-1]-cs[m],0)) * g[n,c,t]
 *                    + sum_{k>=m} exp(min(cs[k]-cs[m],0)) * dy[n,c*Q+k,t].
 * Replaces _chunk_scan_chunk_state_bwd_dx,
 * kernels/ema_kernels_bwd/ema_chunk_scan_chunk_state_bwd_dx.py:208-262. */
int ema_chunk_scan_chunk_state_bwd_dx(const void* dy, int64_t dy_sb, int64_t dy_sl,
                                      int64_t dy_sh, int dtype, const float* cs,
                                      const float* g, void* dx, int64_t dx_sb, int64_t dx_sl,
                                      int64_t dx_sh, int64_t batch, int64_t nheads,
                                      int64_t seqlen, int64_t dim, int64_t chunk,
                                      void* stream);

/* B4: r[m] = exp(min(cs[Q-1]-cs[m],0)) * <g[n,c], x[n,c*Q+m]> written to slot m+1
 * (slot 0 = 0); when raw == 0 an inclusive cumsum along the chunk follows, giving
 * ddA_next[j] = sum_{m<j} r[m].  Output (N,C,Q).
 * Replaces _ema_chunk_state_bwd_db,
 * kernels/ema_kernels_bwd/ema_chunk_state_bwd_db.py:122-152. */
int ema_chunk_state_bwd_db(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh,
                           int dtype, const float* cs, const float* g, float* ddA_next,
                           int raw, int64_t batch, int64_t nheads, int64_t seqlen,
                           int64_t dim, int64_t chunk, void* stream);

/* B5: s[n,c,m] = exp(cs[n,c,m]) * <dy[n,c*Q+m], prev[n,c]> (0 past seqlen).  Output
 * (N,C,Q), before the reverse cumsum.
 * Replaces _ema_chunk_scan_bwd_dC, kernels/ema_kernels_bwd/ema_chunk_scan_bwd_dc.py:115-147. */
int ema_chunk_scan_bwd_dc(const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh,
                          int dtype, const float* prev, const float* cs, float* ddA_prev,
                          int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim,
                          int64_t chunk, void* stream);

/* Bytes of workspace ema_chunk_scan_bwd_ddAcs needs (partial sums per row tile and per column
 * tile, one flag per chunk); 0 for a shape or dtype it does not take. */
size_t ema_chunk_scan_bwd_ddAcs_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen,
                                                int64_t dim, int64_t chunk, int dtype);

/* B6: G[m,k] = exp(min(cs[m]-cs[k],0)) * <dy[m], x[k]> for k < m;
 * ddA_intra[j] = sum_{m>=j} sum_{k<j} G[m,k], ddA_intra[0] = 0.  Output (N,C,Q).
 * Chunks in which cs never rises (every decay) are evaluated in the factored form
 * ddA_intra[j] = exp(cs[j]-cs[j-1]) * <r[j], y[j-1]> with the chunk-local scans y of x and r of dy,
 * in float32: one pass over x and dy for chunks of up to 512 rows, x read twice for longer ones;
 * chunks in which cs rises somewhere by the product itself, with the pairwise minimum.
 * Replaces _ema_chunk_scan_bwd_ddAcs_stable,
 * kernels/ema_kernels_bwd/ema_scan_da.py:113-137. */
int ema_chunk_scan_bwd_ddAcs(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh,
                             const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh,
                             int dtype, const float* cs, float* ddA_intra, void* workspace,
                             size_t workspace_bytes, int64_t batch, int64_t nheads,
                             int64_t seqlen, int64_t dim, int64_t chunk, void* stream);

/* Bytes of workspace ema_bwd_dx_dA_fused needs (per-column-tile partials of ddA). */
size_t ema_bwd_dx_dA_fused_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen,
                                           int64_t dim);

/* B3..B6 and their sum in ONE pass over x and dy, for a chunk size of exactly 128
 * (cs, prev, g are (N, C, 128) / (N, C, T) with C = ceil(seqlen / 128)):
 *   dx[m]  as in B3;
 *   ddA[n,c,m] = exp(A[m]) * <dx[m], y[m-1]>  with y the forward output (y[-1] = prev),
 * which equals ddA_intra + ddA_next + reverse-cumsum(ddA_prev, + ddA_chunk at the last
 * slot): dx[m] is the gradient of the scan state at row m and y[m-1] is the state that
 * exp(A[m]) multiplies.  When y is not NULL the forward output is written there too.
 * The decay of a row is taken as exp(min(cs[m] - cs[m-1], 0)) (cs[-1] = 0 at a chunk's first row).
 * Runs the backward single-pass kernel with both carried states given, so nothing is chained between
 * workgroups and the workspace only holds the partials.
 * Replaces the four launchers _chunk_scan_chunk_state_bwd_dx, _ema_chunk_state_bwd_db,
 * _ema_chunk_scan_bwd_dC, _ema_chunk_scan_bwd_ddAcs_stable and the torch glue around them,
 * kernels/ema_kernels_bwd/ema_combined_bwd.py:70-79. */
int ema_bwd_dx_dA_fused(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, const void* dy,
                        int64_t dy_sb, int64_t dy_sl, int64_t dy_sh, int dtype, const float* cs,
                        const float* prev, const float* g, void* dx, int64_t dx_sb, int64_t dx_sl,
                        int64_t dx_sh, float* ddA, void* y, int64_t y_sb, int64_t y_sl,
                        int64_t y_sh, void* workspace, size_t workspace_bytes, int64_t batch,
                        int64_t nheads, int64_t seqlen, int64_t dim, void* stream);

/* Bytes of workspace ema_bwd needs (cs, states, prev, ds, g and the partial sums). */
size_t ema_bwd_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim,
                               int64_t chunk);

/* Whole backward.  The gradients do not depend on how the sequence is chunked, so the
 * work is done on 128-row chunks in one pass over x and dy: dx, the recomputed forward
 * state and ddA[m] = exp(A[m]) * <dx[m], y[m-1]> per tile, with the reverse inter-chunk
 * state handed from tile to tile inside the kernel (chained scan, last chunk first).
 * `chunk` only fixes the layout of the result.  prev128 (may be NULL) is the output of the
 * same name of ema_fwd; without it the states entering each chunk are recomputed with one
 * more pass over x (F1..F3).  Outputs dx (layout of x) and ddA (N,C,Q) float32 with
 * ddA[n,c,q] = dL/dA[n, c*Q+q] (0 in the slots past seqlen); when y is not NULL the forward
 * output is recomputed into it (the reference's recompute_output=True).  ev_start / ev_stop
 * (hipEvent_t, may be NULL) are recorded right before and after the single-pass kernel.
 * workspace_ready: see the conventions above.
 * Replaces _ema_chunk_scan_combined_bwd,
 * kernels/ema_kernels_bwd/ema_combined_bwd.py:13-83. */
int ema_bwd(const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh, const void* x,
            int64_t x_sb, int64_t x_sl, int64_t x_sh, const float* A, int64_t a_sb,
            int64_t a_sl, int64_t a_sh, const float* prev128, int dtype, void* dx,
            int64_t dx_sb, int64_t dx_sl, int64_t dx_sh, float* ddA, void* y, int64_t y_sb,
            int64_t y_sl, int64_t y_sh, void* workspace, size_t workspace_bytes, int workspace_ready,
            int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim, int64_t chunk, void* stream,
            void* ev_start, void* ev_stop);

/* ------------------------------------------------- sequence-level entry points ---- */

/* Bytes of workspace ema_seq_fwd / ema_seq_bwd need. */
size_t ema_seq_fwd_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim);
size_t ema_seq_bwd_workspace_bytes(int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim);

/* The whole scan in one pass over x, on the caller's raw tensors, with the elementwise steps
 * that the reference's callers run as separate passes folded into the loads and stores:
 *   form = EMA_FORM_LOG_DECAY:   coef = A,  y[t] = exp(min(A[t],0)) * y[t-1] + x[t]
 *   form = EMA_FORM_PROBABILITY: coef = p,  y[t] = (1-p[t]) * y[t-1] + p[t] * x[t]
 *     (the reference forms A = log(1-p) and X = p*x in torch first,
 *      kernels/benchmarks/ema_bench.py:135-136, or runs the three kernels of
 *      ema_scan_combined, kernels/ema.py:370-375)
 * Packed sequences (what the reference's seq_idx arguments ask for, e.g.
 * kernels/ema_chunk_state.py:500-604): the state is dropped at the first position t of a new
 * sequence when A[t] = -inf (log-decay form) or when p[t] carries a set sign bit, i.e. is given
 * as -p[t], -0.0 for p[t] = 0 (probability form; then y[t] = p[t] * x[t]).
 * coef is float32, addressed like A above.  init (N,T) float32, may be NULL = zero: the state
 * before the first position, which the reference's launchers reject
 * (kernels/ema_kernels/ema_state_pass.py:129-130).  final_state (N,T), may be NULL: the state
 * after the last position.  prev128 (N, ceil(seqlen/128), T) float32, required: the state
 * entering each 128-row chunk, which ema_seq_bwd takes.  Chunking is internal; there is no
 * chunk argument.  ev_start / ev_stop and workspace_ready as for ema_fwd.  The call is one
 * kernel launch when the workspace is ready. */
int ema_seq_fwd(int form, const float* coef, int64_t c_sb, int64_t c_sl, int64_t c_sh,
                const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, void* y,
                int64_t y_sb, int64_t y_sl, int64_t y_sh, const float* init, float* final_state,
                float* prev128, void* workspace, size_t workspace_bytes, int workspace_ready,
                int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim, void* stream,
                void* ev_start, void* ev_stop);

/* Backward of ema_seq_fwd in one pass over x and dy.  With r the reverse scan of dy,
 * r[t] = dy[t] + a[t+1] * r[t+1], started from dfinal (N,T) float32 (may be NULL = zero), the
 * gradient reaching final_state:
 *   EMA_FORM_LOG_DECAY:   dx[t] = r[t],        dcoef[t] = a[t] * <r[t], y[t-1]>
 *   EMA_FORM_PROBABILITY: dx[t] = p[t] * r[t], dcoef[t] = <r[t], x[t] - y[t-1]>
 * (at a position whose p carries the sign bit that marks a sequence start, y[t-1] counts as 0 and
 * dcoef[t] is the derivative with respect to the stored value -p[t], i.e. -<r[t], x[t]>)
 * (the reference leaves dP = -dA * exp(A) commented out, kernels/tests/ema_bwd/_ema_full_bwd.py:128-130,
 * and rearranges dA from (b,c,q) to (b,l) in torch, :71).  dcoef is float32 in the layout of
 * coef, given by its own strides; dinit (N,T) float32, may be NULL, receives a[0] * r[0], the
 * gradient of init.  prev128 is the forward's output of that name.  workspace_ready: see the
 * conventions above; the same buffer may serve the forward and the backward call. */
int ema_seq_bwd(int form, const void* dy, int64_t dy_sb, int64_t dy_sl, int64_t dy_sh,
                const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, const float* coef,
                int64_t c_sb, int64_t c_sl, int64_t c_sh, const float* prev128,
                const float* dfinal, int dtype, void* dx, int64_t dx_sb, int64_t dx_sl,
                int64_t dx_sh, float* dcoef, int64_t dc_sb, int64_t dc_sl, int64_t dc_sh,
                float* dinit, void* workspace, size_t workspace_bytes, int workspace_ready,
                int64_t batch, int64_t nheads, int64_t seqlen, int64_t dim, void* stream, void* ev_start,
                void* ev_stop);

/* ------------------------------------------- entry point that allocates nothing ---- */

/* Size of the file-scope device array that ema_seq_fwd_static works in. */
#define EMA_STATIC_SCRATCH_BYTES (16u << 20)
size_t ema_seq_fwd_static_max_workspace_bytes(void);

/* ema_seq_fwd without a workspace argument.  This entry point has no counterpart in the
 * reference; it is for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The status words of the
 * chained scan and the other scratch that ema_seq_fwd takes as `workspace` live in a
 * file-scope device array of EMA_STATIC_SCRATCH_BYTES bytes (one copy per GPU, held until
 * the process ends); the call performs no allocation of any kind, on the device or through a
 * library.  Inputs and outputs are the caller's, with the meaning they have in ema_seq_fwd
 * (prev128 required, init and final_state may be NULL); there is no bwd_workspace and there
 * are no timing events.  Problems whose ema_seq_fwd_workspace_bytes(...) exceeds
 * EMA_STATIC_SCRATCH_BYTES are rejected with EMA_ERR_TOO_LARGE before anything is launched
 * (the b16 nh2 L4096 d1024 problem needs 8.3 MiB).  All calls on one GPU share that GPU's array,
 * which keeps what the last call left in it: the array starts out zero-filled, every call leaves
 * it ready for the next (epoch-tagged words, see the conventions above), so nothing has to be
 * cleared and calls may follow each other on one stream in any order of shapes; calls that
 * overlap in time on one GPU (different streams or threads) race and must be serialised by the
 * caller.  The current device must be the one `stream` belongs to. */
int ema_seq_fwd_static(int form, const float* coef, int64_t c_sb, int64_t c_sl, int64_t c_sh,
                       const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, void* y,
                       int64_t y_sb, int64_t y_sl, int64_t y_sh, const float* init,
                       float* final_state, float* prev128, int64_t batch, int64_t nheads,
                       int64_t seqlen, int64_t dim, void* stream);

/* Companions of ema_seq_fwd_static (no counterpart in the reference either; none of them
 * allocates).
 * ema_seq_fwd_static_init: looks up the device address of the array for the current device
 * (the first look-up on a device may load the code object).  Call it once per device before
 * ema_seq_fwd_static is captured into a HIP graph, so that nothing but kernel launches happens
 * under capture; ema_seq_fwd_static itself does the look-up on its first eager call otherwise.
 * ema_seq_fwd_static_error: copies the sticky error word of the array's chain header to *error
 * (host memory) after synchronising `stream`: non-zero means that some call since the last reset
 * gave up a bounded wait and its outputs hold NaN.
 * ema_seq_fwd_static_reset: zero-fills the array with a kernel on `stream` (the state of a fresh
 * process); needed after an aborted call or a reported error, never in normal operation. */
int ema_seq_fwd_static_init(void);
int ema_seq_fwd_static_error(int* error, void* stream);
int ema_seq_fwd_static_reset(void* stream);

#ifdef __cplusplus
}
#endif
#endif /* EMA_HIP_H */
