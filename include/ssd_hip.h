/*
 * ssd_hip.h -- C ABI of the Mamba-2 SSD chunked-scan forward in libema_hip.so: hand-written
 * HIP kernels for gfx950 (MI355X).
 *
 * Every entry point replaces one launcher of the reference repository
 * kartiksrinivas007/triton-kernels under kernels/mamba_kernels/ (a Python function that
 * allocates its output and starts one Triton kernel); the citation on each declaration is that
 * launcher, with paths relative to the reference root.
 *
 * Conventions (as for ema_hip.h)
 *   - All pointers are DEVICE pointers; the caller allocates inputs and outputs; the library
 *     never allocates, frees or keeps a pointer, and only enqueues work on `stream`.
 *   - x, z, out are (batch, seqlen, nheads, hdim); B, C are (batch, seqlen, ngroups, dstate);
 *     dt is (batch, seqlen, nheads).  Each is addressed as ptr[b*s_b + l*s_l + h*s_h + i] with
 *     strides in ELEMENTS and a unit stride along the last axis.
 *   - Chunked intermediates are dense float32: dt_out and dA_cumsum (batch, nheads, C, Q),
 *     states (batch, C, nheads, hdim, dstate), cb (batch, C, ngroups, Q, Q); C = ceil(seqlen/Q).
 *   - `dtype` (ssd_dtype, same codes as ema_dtype) is the element type of x, z, B, C and out;
 *     accumulation is float32.
 *   - seq_idx (may be NULL) marks a packed batch: int32 ids (batch, seqlen) addressed as
 *     seq_idx[b*seq_sb + l*seq_sl]; positions with different ids belong to different sequences
 *     and do not see each other's state.  Ids are expected to be non-negative and not to
 *     decrease along a row; the carried state of a row starts with id 0.
 *   - Supported shapes: hdim in {64, 128}, dstate in {64, 128}, nheads a multiple of ngroups,
 *     chunk a multiple of 4 up to 1024; anything else returns SSD_ERR_UNSUPPORTED.
 *   - Return value: 0 or a negative ssd_status (same values as ema_status).
 */
#ifndef SSD_HIP_H
#define SSD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  SSD_OK = 0,
  SSD_ERR_NULL = -1,
  SSD_ERR_SHAPE = -2,
  SSD_ERR_ALIGN = -3,
  SSD_ERR_DTYPE = -4,
  SSD_ERR_UNSUPPORTED = -5,
  SSD_ERR_LAUNCH = -6
} ssd_status;

typedef enum { SSD_F32 = 0, SSD_BF16 = 1 } ssd_dtype;

/* dt_out = clamp(softplus?(dt + dt_bias), dt_min, dt_max) (softplus is the identity above 20),
 * 0 past seqlen; dA_cumsum = per-chunk inclusive cumsum of dt_out * A[h].  dt may be float32
 * or bfloat16 (dt_dtype); A and dt_bias (may be NULL) are float32 (nheads).
 * Replaces _chunk_cumsum_fwd, kernels/mamba_kernels/mamba_cumsum.py:103-128. */
int ssd_chunk_cumsum_fwd(const void* dt, int dt_dtype, int64_t dt_sb, int64_t dt_sl, int64_t dt_sh,
                         const float* A, const float* dt_bias, float* dA_cumsum, float* dt_out,
                         int64_t batch, int64_t seqlen, int64_t nheads, int64_t chunk, int dt_softplus,
                         float dt_min, float dt_max, void* stream);

/* states[b,c,h,p,n] = sum_k x[k,p] * B[k,n] * exp(min(dA_last - dA_k, 0)) * dt_k over the
 * positions k of chunk c (the weighted B is rounded to `dtype` before the product, as the
 * reference does).  With seq_idx, position k only counts if its id equals the id of the chunk's
 * last position, and none counts if that id is negative (mamba_state_fwd.py:113).
 * Replaces _chunk_state_fwd, kernels/mamba_kernels/mamba_state_fwd.py:138-169. */
int ssd_chunk_state_fwd(const void* B, int64_t b_sb, int64_t b_sl, int64_t b_sg, const void* x,
                        int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, const float* dt,
                        const float* dA_cumsum, float* states, int64_t batch, int64_t seqlen,
                        int64_t nheads, int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk,
                        const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream);

/* out[b,c] = state entering chunk c; state <- exp(dA_chunk[b,h,c]) * state + states[b,c];
 * final = the state after the last chunk.  states (batch, C, nheads, dim) float32; out the same
 * shape in float32 or bfloat16 (out_dtype: the recurrence itself runs in float32 registers, only
 * the stored copy is rounded, as with out_dtype in mamba_state_pass.py:95-96); final float32;
 * dA_chunk addressed by (batch, head, chunk) strides (it is dA_cumsum[..., -1]); initial
 * (batch, nheads, dim) float32 may be NULL.  dim must be a multiple of 4.  With seq_idx the
 * state is dropped across a chunk whose last position has another id than the previous chunk's
 * last position (id 0 before the first chunk; mamba_state_pass.py:68-71); seqlen and chunk
 * locate those positions and are ignored without seq_idx.
 * Replaces _state_passing_fwd, kernels/mamba_kernels/mamba_state_pass.py:84-115. */
int ssd_state_passing_fwd(const float* states, const float* dA_chunk, int64_t da_sb, int64_t da_sh,
                          int64_t da_sc, const float* initial, void* out, int out_dtype, float* final_states,
                          int64_t batch, int64_t nchunks, int64_t nheads, int64_t dim, const int32_t* seq_idx,
                          int64_t seq_sb, int64_t seq_sl, int64_t seqlen, int64_t chunk, void* stream);

/* ssd_chunk_state_fwd and ssd_state_passing_fwd in one pass over x and B: the chunk-local states,
 * which are float32 and twice the bytes of x, stay in registers instead of going through memory.
 * out (batch, C, nheads, hdim, dstate), float32 or bfloat16 (out_dtype), receives the state entering
 * each chunk; final_states (batch, nheads, hdim, dstate) float32 the state after the last chunk;
 * initial of that shape, float32, may be NULL.  The results equal those of the two entry points
 * called one after the other bit for bit.  chunk must be a multiple of 64 (SSD_ERR_UNSUPPORTED
 * otherwise); packed batches (seq_idx) go through the two separate entry points.
 * Replaces the pair _chunk_state_fwd, kernels/mamba_kernels/mamba_state_fwd.py:138-169, and
 * _state_passing_fwd, kernels/mamba_kernels/mamba_state_pass.py:84-115, where a caller runs them
 * back to back (the single-kernel chunk walk of kernels/mamba_3_kernels/mamba_ssd_fwd.py:247-258
 * carries its state the same way). */
int ssd_chunk_state_passing_fwd(const void* B, int64_t b_sb, int64_t b_sl, int64_t b_sg, const void* x,
                                int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype, const float* dt,
                                const float* dA_cumsum, const float* initial, void* out, int out_dtype,
                                float* final_states, int64_t batch, int64_t seqlen, int64_t nheads,
                                int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk, void* stream);

/* out[b,c,g,m,k] = sum_n a[b,cQ+m,g,n] * bm[b,cQ+k,g,n]; rows past seqlen are zero.  out is
 * float32 or `dtype` (out_dtype).  With seq_idx, out[m,k] = 0 where the ids of m and k differ
 * (mamba_bmm.py:70-73).  Replaces _bmm_chunk_fwd, kernels/mamba_kernels/mamba_bmm.py:88-126
 * (the whole Q x Q block is written, also with causal = True). */
int ssd_bmm_chunk_fwd(const void* a, int64_t a_sb, int64_t a_sl, int64_t a_sg, const void* bm,
                      int64_t b_sb, int64_t b_sl, int64_t b_sg, int dtype, void* out, int out_dtype,
                      int64_t batch, int64_t seqlen, int64_t ngroups, int64_t k, int64_t chunk,
                      const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream);

/* out[m,p] = exp(dA_m) * sum_n C[m,n] * prev[p,n]
 *          + sum_{k<=m} cb[m,k] * exp(min(dA_m - dA_k, 0)) * dt_k * x[k,p]  +  D * x[m,p],
 * then, with z: out_x = out (if out_x is not NULL) and out *= z * sigmoid(z).
 * cb float32 (batch, C, ngroups, Q, Q); prev (batch, C, nheads, hdim, dstate) in float32 or in
 * `dtype` (states_dtype; the product rounds it to `dtype` either way, so the result is the same and
 * the bfloat16 form moves half the bytes); D float32
 * (nheads) or (nheads, hdim) (d_has_hdim), may be NULL; z may be NULL; out_x shares out's strides.
 * With seq_idx the first term only reaches the rows m whose id equals that of the previous
 * chunk's last position (0 for the first chunk; mamba_scan_fwd.py:77-92); cb is expected to
 * hold zeros between positions of different ids, as ssd_bmm_chunk_fwd leaves it.
 * Replaces _chunk_scan_fwd, kernels/mamba_kernels/mamba_scan_fwd.py:162-210. */
int ssd_chunk_scan_fwd(const float* cb, const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh,
                       const void* z, int64_t z_sb, int64_t z_sl, int64_t z_sh, int dtype,
                       const float* dt, const float* dA_cumsum, const void* C, int64_t c_sb, int64_t c_sl,
                       int64_t c_sg, const void* prev_states, int states_dtype, const float* D, int d_has_hdim,
                       void* out, int64_t o_sb, int64_t o_sl, int64_t o_sh, void* out_x, int64_t batch,
                       int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t hdim, int64_t dstate,
                       int64_t chunk, const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream);

/* ---------------------------------------------------------------- backward stages ---- */

/* dprev_states[b,c,h,p,n] = sum_m round(dout[m,p] * exp(dA_m)) * C[m,n]: the gradient of the chunk
 * scan with respect to the carried states, accumulated in float32 and stored in float32 or in
 * `dtype` (states_dtype; the dtype argument of the reference's launcher).  With seq_idx only the rows m whose id
 * equals that of the previous chunk's last position count (mamba_scan_bwd.py:63-71).
 * Replaces _chunk_scan_bwd_dstates,
 * kernels/mamba_kernels_bwd/mamba_scan_bwd.py:91-116. */
int ssd_chunk_scan_bwd_dstates(const void* C, int64_t c_sb, int64_t c_sl, int64_t c_sg, const void* dout,
                               int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype, const float* dA_cumsum,
                               void* dprev_states, int states_dtype, int64_t batch, int64_t seqlen,
                               int64_t nheads, int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk,
                               const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream);

/* Bytes of workspace ssd_state_passing_bwd needs (per-wave partial dot products). */
size_t ssd_state_passing_bwd_workspace_bytes(int64_t batch, int64_t nchunks, int64_t nheads, int64_t dim);

/* Reverse inter-chunk recurrence.  states (batch, C, nheads, dim) are the states ENTERING each
 * chunk (index 0 the initial one), dout the gradient with respect to them, dfinal (may be NULL)
 * the gradient of the final state.  With G the gradient of the state entering the next chunk:
 * dstates[c] = G (the gradient of the chunk-local state), ddA_chunk[b,h,c] = exp(dA_chunk[c]) *
 * <states[c], G> (0 for c = 0 unless dinit is given), G <- exp(dA_chunk[c]) * G + dout[c];
 * dinit (batch, nheads, dim), may be NULL, receives the last G.  All float32, except that states,
 * dout and dstates may each be bfloat16 (states_dtype, dout_dtype, dstates_dtype, as with
 * dstates_dtype / states_dtype in the reference's launcher; G itself stays in float32 registers).
 * With seq_idx the
 * factor exp(dA_chunk[c]) is 0 for the chunks across which ssd_state_passing_fwd drops the state
 * (mamba_state_passing_bwd_dstates.py:72-80,105); seqlen and chunk as there.
 * Replaces _state_passing_bwd, kernels/mamba_kernels_bwd/mamba_state_passing_bwd_dstates.py:116-172. */
int ssd_state_passing_bwd(const void* states, int states_dtype, const float* dA_chunk, int64_t da_sb, int64_t da_sh,
                          int64_t da_sc, const void* dout, int dout_dtype, const float* dfinal, void* dstates,
                          int dstates_dtype,
                          float* ddA_chunk, float* dinit, void* workspace, size_t workspace_bytes,
                          int64_t batch, int64_t nchunks, int64_t nheads, int64_t dim, const int32_t* seq_idx,
                          int64_t seq_sb, int64_t seq_sl, int64_t seqlen, int64_t chunk, void* stream);

/* Bytes of workspace ssd_chunk_scan_state_passing_bwd needs (per-wave partial dot products). */
size_t ssd_chunk_scan_state_passing_bwd_workspace_bytes(int64_t batch, int64_t nchunks, int64_t nheads);

/* ssd_chunk_scan_bwd_dstates followed by ssd_state_passing_bwd in one kernel (no counterpart among
 * the reference's launchers, the mirror image of ssd_chunk_state_passing_fwd): a workgroup per
 * (batch, head) walks the chunks from the last to the first, forms the chunk's gradient with respect
 * to its entering state in the accumulators and feeds it to the reverse recurrence there, so that
 * this state-sized float32 tensor is neither written nor read back.  C, dout, dA_cumsum as for
 * ssd_chunk_scan_bwd_dstates; states, dfinal, dstates, ddA_chunk, dinit as for ssd_state_passing_bwd
 * (dim = hdim * dstate, dA_chunk = dA_cumsum[..., chunk - 1]).  The results are those of the two
 * entry points called one after the other with a float32 tensor between them: dstates bit for bit,
 * ddA_chunk up to the order of its sums.  Written for bfloat16 dout / C / states, hdim 64,
 * dstate 128, chunk a multiple of 64 and at least 128, non-negative strides; anything else, and a
 * packed batch (seq_idx), returns SSD_ERR_UNSUPPORTED and goes through the two separate entry points.
 * Replaces the pair _chunk_scan_bwd_dstates, kernels/mamba_kernels_bwd/mamba_scan_bwd.py:91-116, and
 * _state_passing_bwd, kernels/mamba_kernels_bwd/mamba_state_passing_bwd_dstates.py:116-172, where a
 * caller runs them back to back. */
int ssd_chunk_scan_state_passing_bwd(const void* C, int64_t c_sb, int64_t c_sl, int64_t c_sg, const void* dout,
                                     int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype, const float* dA_cumsum,
                                     const void* states, int states_dtype, const float* dfinal, void* dstates,
                                     int dstates_dtype, float* ddA_chunk, float* dinit, void* workspace,
                                     size_t workspace_bytes, int64_t batch, int64_t seqlen, int64_t nheads,
                                     int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk, void* stream);

/* dB[b,l,g,n] = sum over the heads h of group g of (sum_p x[m,p] * round(dstates[b,c,h,p,n])) *
 * exp(min(dA_last - dA_m, 0)) * dt_m (float32, dense (batch, seqlen, ngroups, dstate)).  With B
 * (may be NULL, then ddA_cumsum is not written): r_h[m] = sum_n db_h[m,n] * B[m,n] and
 * ddA_cumsum[b,h,c,j] = sum_{m<j} r_h[m], the gradient of the chunk states with respect to the
 * per-position dA.  With seq_idx the weight of row m is 0 unless its id equals that of the
 * chunk's last position (mamba_chunk_state_bwd_db.py:88-104).  dstates in float32 or in `dtype`
 * (states_dtype).  Replaces _chunk_state_bwd_db,
 * kernels/mamba_kernels_bwd/mamba_chunk_state_bwd_db.py:131-181 (one pass over all heads of a
 * group, so there is no split axis to sum afterwards). */
int ssd_chunk_state_bwd_db(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, int dtype,
                           const float* dt, const float* dA_cumsum, const void* dstates, int states_dtype,
                           const void* B, int64_t b_sb, int64_t b_sl, int64_t b_sg, float* dB, float* ddA_cumsum,
                           int64_t batch, int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t hdim,
                           int64_t dstate, int64_t chunk, const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl,
                           void* stream);

/* dC[b,l,g,n] = sum over the heads of group g of (sum_p dout[m,p] * round(prev[b,c,h,p,n])) *
 * exp(dA_m): the part of dC that comes through the carried state.  With C (may be NULL):
 * ddA_cumsum_prev[b,h,c,m] = sum_n dc_h[m,n] * C[m,n].  With seq_idx the weight of row m is 0
 * unless its id equals that of the previous chunk's last position
 * (mamba_chunk_scan_bwd_dc.py:84-96).  prev_states in float32 or in `dtype` (states_dtype), as
 * for ssd_chunk_scan_fwd.  Replaces _chunk_scan_bwd_dC,
 * kernels/mamba_kernels_bwd/mamba_chunk_scan_bwd_dc.py:118-160. */
int ssd_chunk_scan_bwd_dc(const void* dout, int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype,
                          const float* dA_cumsum, const void* prev_states, int states_dtype, const void* C,
                          int64_t c_sb, int64_t c_sl, int64_t c_sg, float* dC, float* ddA_cumsum_prev, int64_t batch,
                          int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t hdim, int64_t dstate,
                          int64_t chunk, const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, void* stream);

/* acc[m,p] = exp(min(dA_last - dA_m, 0)) * sum_n B[m,n] * round(dstates[p,n])
 *          + sum_{k>=m} round(cb[k,m] * exp(min(dA_k - dA_m, 0))) * dout[k,p];
 * dx = acc * dt_m + D * dout (type `dtype`, dx's own strides), ddt[b,h,c,m] = sum_p acc[m,p] * x[m,p]
 * (float32, 0 past seqlen).  cb float32 (batch, C, ngroups, Q, Q), dstates float32 or `dtype`
 * (states_dtype) (batch, C, nheads, hdim, dstate), D as for ssd_chunk_scan_fwd.  dD_partial (may be NULL; needs D):
 * float32 (batch, C, nheads, S, hdim) with S = ssd_chunk_scan_chunk_state_bwd_dx_dD_slots(...),
 * every slot written: partial sums over positions of dout * x, whose sum over batch, C and S is
 * the gradient of D (nheads, hdim), summed over hdim too for a D of shape (nheads) -- the
 * reference writes such partials per block and sums them in torch
 * (mamba_chunk_scan_chunk_state_bwd_dx.py:176-183,245-247).  With seq_idx the first term only reaches the rows m whose id equals that
 * of the chunk's last position (mamba_chunk_scan_chunk_state_bwd_dx.py:93-96).
 * Replaces _chunk_scan_chunk_state_bwd_dx,
 * kernels/mamba_kernels_bwd/mamba_chunk_scan_chunk_state_bwd_dx.py:189-248. */
int ssd_chunk_scan_chunk_state_bwd_dx(const float* cb, const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh,
                                      const void* dout, int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype,
                                      const float* dt, const float* dA_cumsum, const void* B, int64_t b_sb,
                                      int64_t b_sl, int64_t b_sg, const void* dstates, int states_dtype, const float* D,
                                      int d_has_hdim, void* dx, int64_t dx_sb, int64_t dx_sl, int64_t dx_sh,
                                      float* ddt, int64_t batch, int64_t seqlen, int64_t nheads,
                                      int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk,
                                      const int32_t* seq_idx, int64_t seq_sb, int64_t seq_sl, float* dD_partial,
                                      void* stream);

/* Slots per (batch, chunk, head) of dD_partial above for a shape; 0 for an unsupported one. */
int64_t ssd_chunk_scan_chunk_state_bwd_dx_dD_slots(int dtype, int64_t hdim, int64_t dstate, int64_t chunk);

/* Bytes of workspace ssd_chunk_scan_bwd_ddAcs needs (column sums per row tile, row sums). */
size_t ssd_chunk_scan_bwd_ddAcs_workspace_bytes(int64_t batch, int64_t seqlen, int64_t nheads, int64_t chunk);

/* With W[m,n] = <dout[m], x[n]> * dt_n * cb[m,n] * exp(min(dA_m - dA_n, 0)) for n < m:
 * ddA_cumsum[b,h,c,j] = sum_{m>=j} sum_{n<j} W[m,n] (float32; 0 for j = 0): the gradient of the causal
 * term of the chunk scan with respect to the per-position dA.  It is formed as the prefix sum of
 * (column sum - row sum) of W, which is the same quantity as the reference's row-wise cumsum
 * followed by column sums.  A packed batch needs nothing here: cb already holds zeros between
 * positions of different ids (mamba_chunk_scan_bwd_da.py:86).  Replaces _chunk_scan_bwd_ddAcs_stable,
 * kernels/mamba_kernels_bwd/mamba_chunk_scan_bwd_da.py:111-140 (and its torch sum over row blocks). */
int ssd_chunk_scan_bwd_ddAcs(const void* x, int64_t x_sb, int64_t x_sl, int64_t x_sh, const void* dout,
                             int64_t d_sb, int64_t d_sl, int64_t d_sh, int dtype, const float* dt,
                             const float* dA_cumsum, const float* cb, float* ddA_cumsum, void* workspace,
                             size_t workspace_bytes, int64_t batch, int64_t seqlen, int64_t nheads,
                             int64_t ngroups, int64_t hdim, int64_t chunk, void* stream);

/* States at the end of each sequence of a packed batch (batch dimension 1, sequences back to
 * back): cu_seqlens (nseq + 1, int32, device memory) holds the first position of each sequence and
 * the total length.  B (seqlen, ngroups, dstate) and x (seqlen, nheads, hdim) with element strides
 * for position and group / head (innermost contiguous); dt, dA_cumsum (nheads, nchunks, chunk)
 * float32 contiguous; chunk_states (nchunks, nheads, hdim, dstate) contiguous, float32 or `dtype`
 * (states_dtype), the state entering each chunk (what ssd_state_passing_fwd writes).  states (nseq, nheads, hdim, dstate)
 * float32 is written in full; a sequence of length 0, or bounds outside [0, seqlen], give zeros.
 * Any hdim and dstate up to 4096.  For sequence s ending (exclusive) at e in chunk c = (e-1)/chunk:
 *   states[s] = sum_{k in s, k in chunk c} exp(min(dA[e-1] - dA[k], 0)) dt[k] x[k] (outer) B[k]
 *             + (s began before chunk c) * exp(dA[e-1]) * chunk_states[c].
 * Replaces chunk_state_varlen, kernels/ema_chunk_state.py:578-604 (kernel at :500-575). */
int ssd_chunk_state_varlen(const void* B, int64_t b_sl, int64_t b_sg, const void* x, int64_t x_sl, int64_t x_sh,
                           int dtype, const float* dt, const float* dA_cumsum, const void* chunk_states,
                           int states_dtype, const int32_t* cu_seqlens, float* states, int64_t nseq, int64_t seqlen, int64_t nheads,
                           int64_t ngroups, int64_t hdim, int64_t dstate, int64_t chunk, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SSD_HIP_H */
