/*
 * spion_hip.h -- C ABI of libspion_hip.so: SPION layer-wise sparse attention for AMD MI355X (gfx950).
 *
 * Every pointer argument is a DEVICE pointer unless a comment says "host".  float = IEEE fp32,
 * int = int32.  The caller owns every buffer it passes (inputs, outputs and the dP / dS scratch
 * arrays); the library owns only the handle and the private workspace hanging off it.  All work is
 * enqueued on the handle's stream (the HIP null stream unless spion_set_stream was called), which is
 * the stream PyTorch-ROCm uses by default, so results are ordered with the surrounding torch ops and
 * no call synchronises the host in steady state.  The first call that sees a new (Offsets, Columns,
 * nnz) triple copies the index to the host once to analyse it (tile detection, transposed index).
 *
 * The four entry points of each family have the signatures the reference's ctypes declarations bind
 * (reference: models/attention.py:141-191); the drop-in libraries attn.so, attn_mask.so,
 * block_attn.so and block_attn_mask.so re-export them under the reference's un-prefixed names
 * init / attn_forward / attn_backward / destroy.
 *
 * Like the reference, the attention entry points return void.  Failures (bad handle, inconsistent
 * CSR, HIP errors) are recorded and can be read with spion_last_error(); after a failure the call
 * launches nothing.
 */
#ifndef SPION_HIP_H
#define SPION_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------------
 * Sparse attention on an element-level CSR pattern, no key mask.
 * Replaces models/block_attn.cu:547-568 (init / attn_forward / attn_backward / destroy).
 *
 *   NB = num_batches = batch * heads,  L = seq_len,  d = emb_dim,  n = nnz per (batch, head).
 *   Offsets[L+1]  exclusive prefix sum of per-row counts, shared by all NB problems.
 *   Columns[>=n]  sorted column indices per row; only the first n entries are read (the reference
 *                 passes NB identical copies, models/attention_blockcuda.py:43).
 *   SumMat[L]     per-row counts (= Offsets[i+1]-Offsets[i]); accepted for compatibility, not read.
 *   Attn[NB*n]    out: probabilities P in CSR order, problem stride n.
 *
 * Semantics (models/block_attn.cu:33-88): off-pattern logits count as 0 in the softmax denominator:
 *   v = (q_i . k_j)/sqrt(d);  m = max(-100, max_j v);  Z = sum_j exp(v-m) + (L-n_i) exp(-m);  P = exp(v-m)/Z.
 * ---------------------------------------------------------------------------------------------- */
void* spion_block_init(int emb_dim, int seq_len, int num_batches, int block_size);

/* Q [NB][L][d], Kt [NB][d][L] (K transposed), V [NB][L][d]; out: Attn [NB*n], Out [NB][L][d].
 * Reference: models/block_attn.cu:552-556. */
void spion_block_attn_forward(void* handle, const float* Q, const float* Kt, const float* V,
                              float* Attn, float* Out,
                              const int* Offsets, const int* Columns, const int* SumMat, int nnz);

/* Q, K [NB][L][d], Vt [NB][d][L] (V transposed), P = Attn of the forward, dO [NB][L][d];
 * dP, dS: caller-owned scratch of NB*n floats each, contents unspecified on return;
 * out: dQ, dK, dV [NB][L][d] (need not be zeroed).  Reference: models/block_attn.cu:558-563. */
void spion_block_attn_backward(void* handle, const float* Q, const float* K, const float* Vt,
                               const float* P, const float* dO, float* dP, float* dS,
                               float* dQ, float* dK, float* dV,
                               const int* Offsets, const int* Columns, const int* SumMat, int nnz);

void spion_block_destroy(void* handle);

/* ------------------------------------------------------------------------------------------------
 * Sparse attention on an element-level CSR pattern with an additive key-padding penalty.
 * Replaces models/block_attn_mask.cu:655-674.
 *   Mask[NB*L]: 0 for valid keys, 1e6 for padded keys, index (b*H+h)*L + key
 *   (models/attention_blockcuda_mask.py:42-43).
 *   v = (q_i . k_j)/sqrt(d) - Mask[bh*L + j];  m = max(0, max_j v)  (models/block_attn_mask.cu:88-140).
 * ---------------------------------------------------------------------------------------------- */
void* spion_blockmask_init(int emb_dim, int seq_len, int num_batches, int block_size);

void spion_blockmask_attn_forward(void* handle, const float* Q, const float* Kt, const float* V,
                                  const float* Mask, float* Attn, float* Out,
                                  const int* Offsets, const int* Columns, const int* SumMat, int nnz);

void spion_blockmask_attn_backward(void* handle, const float* Q, const float* K, const float* Vt,
                                   const float* P, const float* dO, float* dP, float* dS,
                                   float* dQ, float* dK, float* dV,
                                   const int* Offsets, const int* Columns, const int* SumMat, int nnz);

void spion_blockmask_destroy(void* handle);

/* ------------------------------------------------------------------------------------------------
 * Sparse attention on bf16 tensors (scale-up shapes).  No counterpart in the reference, which is fp32 only;
 * the arithmetic is that of models/block_attn.cu:33-130 (with Mask: models/block_attn_mask.cu:88-173) on
 * bf16 inputs with fp32 accumulation and softmax.  Like the reference's key-mask module
 * (models/attention_blockcuda_mask.py:61, which returns 0 for the map) it does not hand out the probabilities:
 * they are never written to memory, the backward recomputes them.
 *   Q, K, V, Out, dO, dQ, dK, dV: bf16, row-major [NB][L][d] (no transposed operands), d = 32 or 64;
 *   Mask: NULL, or the additive key penalty [NB][L] fp32 of the block-mask family;
 *   Lse [NB][L] fp32: written by the forward (row maximum + log2 of the softmax denominator, log2 domain),
 *     to be handed back to the backward together with Out;
 *   the pattern must be a union of aligned 32x32 tiles (any block mask with block size 32, 64, ...).
 * ---------------------------------------------------------------------------------------------- */
void* spion_block_bf16_init(int emb_dim, int seq_len, int num_batches, int block_size);

void spion_block_bf16_attn_forward(void* handle, const void* Q, const void* K, const void* V, const float* Mask,
                                   void* Out, float* Lse,
                                   const int* Offsets, const int* Columns, const int* SumMat, int nnz);

void spion_block_bf16_attn_backward(void* handle, const void* Q, const void* K, const void* V, const float* Mask,
                                    const void* Out, const float* Lse, const void* dO,
                                    void* dQ, void* dK, void* dV,
                                    const int* Offsets, const int* Columns, const int* SumMat, int nnz);

void spion_block_bf16_destroy(void* handle);

/* ------------------------------------------------------------------------------------------------
 * Dense-phase attention (produces the full probability map that feeds pattern discovery).
 * Replaces models/attn.cu:265-280.  Operands follow the reference's column-major convention:
 *   forward : Qt [NB][d][L], K [NB][L][d], Vt [NB][d][L];
 *             out Attn [NB][L(key)][L(query)] (Attn[h][j][i] = P[i][j]), Out [NB][d][L].
 *   backward: Qt, Kt [NB][d][L], V [NB][L][d], P = Attn, dOt [NB][d][L];
 *             dP, dScale, dS: caller scratch [NB][L][L] (dScale is never touched);
 *             out dQ, dK, dV as [NB][d][L].
 *   v = (q_i . k_j)/sqrt(d);  m = max(-10, max_j v);  P = softmax_j  (models/attn.cu:9-36).
 * ---------------------------------------------------------------------------------------------- */
void* spion_dense_init(int emb_dim, int seq_len, int num_batches);

void spion_dense_attn_forward(void* handle, const float* Qt, const float* K, const float* Vt,
                              float* Attn, float* Out);

void spion_dense_attn_backward(void* handle, const float* Qt, const float* Kt, const float* V,
                               const float* P, const float* dOt, float* dP, float* dScale, float* dS,
                               float* dQ, float* dK, float* dV);

void spion_dense_destroy(void* handle);

/* Dense-phase attention with the key-padding penalty Mask[NB*L] subtracted from the logits.
 * Replaces models/attn_mask.cu:280-298. */
void* spion_densemask_init(int emb_dim, int seq_len, int num_batches);

void spion_densemask_attn_forward(void* handle, const float* Qt, const float* K, const float* Vt,
                                  const float* Mask, float* Attn, float* Out);

void spion_densemask_attn_backward(void* handle, const float* Qt, const float* Kt, const float* V,
                                   const float* P, const float* dOt, float* dP, float* dScale, float* dS,
                                   float* dQ, float* dK, float* dV);

void spion_densemask_destroy(void* handle);

/* ------------------------------------------------------------------------------------------------
 * Pattern discovery on the device.  The reference does this in Python on the host CPU
 * (main_conv_ff.py:254-278, main_conv.py:236-256, main_ff.py:253-272); there is no reference FFI.
 *
 *   Score  [n_maps][L][L]  head/batch-averaged probability maps (one per layer).
 *   Mat    [n_maps][nb][nb] out: 0.0 / 1.0 block masks, nb = L / block_size.
 *   Pooled [n_maps][nb][nb] out, optional (may be NULL): pooled filtered map, fp32.  With NULL the library
 *                           uses one buffer of its own, shared by all such calls: callers that run
 *                           discovery on several streams at once pass their own Pooled.
 *   Thresh [n_maps]         out, optional (may be NULL): the quantile threshold used.
 *   conv_ksize : odd size of the diagonal (identity) filter, 31 in the reference; 0 = no filter.
 *   mode       : SPION_PATTERN_FLOOD  -> param = quantile q in [0,1], greedy path walk from the
 *                                        top row and left column, then the diagonal is set;
 *                SPION_PATTERN_TOPK   -> param = density; the int(nb*nb*density - nb) largest
 *                                        pooled blocks (ties: lower index first), then the diagonal.
 *   stream     : a hipStream_t, or NULL for the null stream.
 * Filter and pooling accumulate in fp64 and round once to fp32.  Returns 0 on success.
 * ---------------------------------------------------------------------------------------------- */
#define SPION_PATTERN_FLOOD 0
#define SPION_PATTERN_TOPK 1

int spion_pattern_generate(const float* Score, int n_maps, int seq_len, int block_size,
                           int conv_ksize, int mode, double param,
                           float* Mat, float* Pooled, float* Thresh, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Score map of a layer for pattern discovery: the mean of the dense phase's probability maps over the
 * batch and then over the heads -- models/model_transformer.py:136-137
 * (attn_lst.append(torch.mean(torch.mean(attn, dim=0), dim=0))) -- in one pass over the maps.
 *   Attn [batch][heads][seq_len][seq_len] fp32 device memory.  key_major != 0: every map is stored
 *        keys x queries, the layout the dense attn_forward writes (models/attention_cuda.py:30-44 hands
 *        it out as a permuted view); key_major == 0: queries x keys.
 *   Mean [seq_len][seq_len] out, queries x keys: the Score input of spion_pattern_generate.
 * seq_len must be a multiple of 32.  Returns 0 on success.
 * ---------------------------------------------------------------------------------------------- */
int spion_score_map_mean(const float* Attn, int batch, int heads, int seq_len, int key_major,
                         float* Mean, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Dense-to-sparse transition test on the device (main_conv_ff.py:211-242; the reference runs it on the host
 * with one synchronising torch reduction per layer).  Call once per evaluation with the averaged score maps of all
 * layers; the decision accumulates in State and is read back by the caller as one float.
 *   Cur     [layers][elems_per_layer]  this evaluation's maps;
 *   Prev    [layers][elems_per_layer]  in/out: the maps kept for comparison (contents need not be initialised);
 *   State   [2*layers + 3] floats, in/out, zero-initialised by the caller before the first call:
 *           [0, layers)            Frobenius distance of the previous comparison, per layer
 *           [layers, 2*layers)     last change of the distance in per cent, per layer
 *           [2*layers]             stage: 0 no map kept yet, 1 maps kept, 2 maps and distances kept
 *           [2*layers + 1]         1 once the change stayed below `percent` (truncated to an integer, as the
 *                                  reference's int(diff) < 15) in every layer; later calls change nothing
 *           [2*layers + 2]         scratch
 *   Partial [layers][partial_blocks] doubles: workspace.
 * First call: the maps are kept.  Second call: the first distances are taken, the kept maps stay.  Later calls:
 * the distance to the kept maps is compared with the previous distance; if not every layer has settled, the kept
 * maps are replaced by the current ones.  Differences are formed in fp32 as torch does, summed in fp64 in a fixed
 * order.  Returns 0 on success. */
int spion_transition_update(const float* Cur, float* Prev, int layers, long long elems_per_layer,
                            float* State, double* Partial, int partial_blocks, int percent, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Additions with no counterpart in the reference (which reports no errors at all).
 * ---------------------------------------------------------------------------------------------- */

/* Message of the most recent failure in this process, or "" if none since spion_clear_error(). */
const char* spion_last_error(void);
void spion_clear_error(void);
/* 1 if spion_last_error() would return a message, else 0: the cheap check for a caller that polls after every
 * call. */
int spion_error_pending(void);

/* Launch this handle's work on `stream` (a hipStream_t; NULL = null stream).  Any family. */
void spion_set_stream(void* handle, void* stream);

/* The analysis of a pattern (tile detection, transposed index) is cached per handle under the key
 * (Offsets pointer, Columns pointer, nnz), up to 8 patterns per handle, least recently used evicted.  The key
 * says nothing about the arrays' contents.  A caller that frees index arrays, or rewrites them in place, MUST
 * drop the key before the addresses can carry another pattern -- with spion_forget_pattern for that one pair of
 * arrays, or spion_invalidate_pattern for everything the handle holds; otherwise a later pattern at the same
 * addresses with the same nnz silently runs on the old index.  (The Python modules do this when their mask
 * cache evicts an entry.) */
void spion_invalidate_pattern(void* handle);
void spion_forget_pattern(void* handle, const int* Offsets, const int* Columns);

/* Analyse a pattern ahead of its first use from HOST copies of the index arrays (host_Offsets [L+1],
 * host_Columns [nnz]: host pointers) and file it under the device arrays Offsets / Columns: the first
 * attn_forward with that pair then copies nothing back to the host and does not wait for the stream -- what a
 * loader of saved masks does once per mask (the reference rebuilds the index on every forward,
 * models/attention_blockcuda.py:26-43, and loads masks in main_inference.py:164-172).  Also the way to make a
 * pattern known before a HIP graph capture.  Returns 0 on success; on a
 * malformed index nothing is filed and the error is recorded. */
int spion_register_pattern(void* handle, const int* Offsets, const int* Columns, int nnz,
                           const int* host_Offsets, const int* host_Columns);

/* Which kernel family the last forward/backward of a sparse handle used:
 * 0 = none yet, 1 = MFMA 32x32 tile path, 2 = element (gather) path, 3 = hybrid path (element-sparse pattern
 * whose well-filled 32x32 tiles run on the MFMA units, the rest on the gather kernels).  For 2 and 3 the backward
 * needs the dS scratch.  It describes the most recent call on the handle, not a particular pattern. */
int spion_last_path(void* handle);

/* Most recent failure recorded by a call on THIS handle ("" if none), besides the process-wide slot of
 * spion_last_error, which any thread or handle can overwrite.  Every failure is also written to stderr unless
 * the environment has SPION_QUIET=1; SPION_ABORT_ON_ERROR=1 makes a failure abort the process (for callers of the
 * void-returning drop-in symbols, who have no other signal). */
const char* spion_handle_error(void* handle);
void spion_clear_handle_error(void* handle);

/* The forward of the MFMA tile path keeps a private copy of Out, filed under the Attn pointer it filled
 * (up to 4 per handle, NB*L*d floats each); a backward given the same P pointer then gets its softmax
 * row sums from dO.Out in one step.  on = 0 switches the copies off (the backward then recomputes the
 * row sums with one more sweep over the tiles); default on. */
void spion_use_output_cache(void* handle, int on);

/* attn_backward of the two sparse families (spion_block_* and spion_blockmask_*) for callers that still hold
 * the forward's output -- the reference's backward (models/block_attn.cu:558) is not handed it.  Out
 * [NB][L][d] fp32: the row sums dO.Out come from it, so such callers can switch the kept copies off
 * (spion_use_output_cache(handle, 0)) and save their memory and traffic.  All other arguments as in
 * spion_block_attn_backward. */
void spion_attn_backward_with_out(void* handle, const float* Q, const float* K, const float* Vt, const float* P,
                                  const float* Out, const float* dO, float* dP, float* dS,
                                  float* dQ, float* dK, float* dV,
                                  const int* Offsets, const int* Columns, const int* SumMat, int nnz);

/* The sparse entry points for callers whose tensors are all row-major [NB][L][d] -- the layout the reference's
 * modules start from before they make the transposed copies its ABI asks for
 * (models/attention_blockcuda.py:48 key.permute(0,1,3,2), :80 value.permute(0,1,3,2)).  K (forward) and V
 * (backward) are read as they are: no transposed copy is made by anyone (d = 32 and the element kernels; the
 * d = 64 tile kernels make one internally).  Mask: NULL for a handle of spion_block_init, the [NB][L] penalty
 * for a handle of spion_blockmask_init.  Out in the backward: the forward's output (may be NULL: the kept copy,
 * or one more sweep, is used).  dS: scratch [NB][nnz] floats, needed for patterns that are not made of aligned
 * 32x32 tiles (element and hybrid kernels; contents unspecified on return); may be NULL for tile patterns. */
void spion_attn_forward_rowmajor(void* handle, const float* Q, const float* K, const float* V, const float* Mask,
                                 float* Attn, float* Out,
                                 const int* Offsets, const int* Columns, const int* SumMat, int nnz);
void spion_attn_backward_rowmajor(void* handle, const float* Q, const float* K, const float* V, const float* P,
                                  const float* Out, const float* dO, float* dS,
                                  float* dQ, float* dK, float* dV,
                                  const int* Offsets, const int* Columns, const int* SumMat, int nnz);

/* spion_attn_backward_rowmajor for callers that cannot allocate.  No counterpart in the reference; it is for
 * callers that cannot call hipMalloc: code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation.  Same arguments and results (bit for bit) as spion_attn_backward_rowmajor with Out given, minus the
 * dS scratch; it calls no hipMalloc / hipFree and no allocating library routine.  The row sums the row pass
 * leaves for the column pass go to a built-in device array of spion_noalloc_max_rows() floats (2^20 = 4 MiB,
 * held by every GPU the library runs on until the process ends) instead of the handle's workspace.
 * Limits, each reported through the error slot with nothing launched:
 *   num_batches * seq_len <= spion_noalloc_max_rows();  emb_dim 32;  Out required;
 *   the pattern must be a union of aligned 32x32 tiles and must already be analysed on this handle
 *   (by an earlier forward with the same Offsets / Columns / nnz, or by spion_register_pattern).
 * All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads, two handles)
 * race.  Nothing in it needs clearing between calls: the row pass writes every row sum the column pass reads. */
void spion_attn_backward_noalloc(void* handle, const float* Q, const float* K, const float* V, const float* P,
                                 const float* Out, const float* dO,
                                 float* dQ, float* dK, float* dV,
                                 const int* Offsets, const int* Columns, const int* SumMat, int nnz);
long long spion_noalloc_max_rows(void);

/* The same for heads that are views of other memory: the reference's layer produces Q, K and V as
 * [B][L][H*d] projections and views them as [B][H][L][d] (models/attention.py:84-96 and split_heads :136-139),
 * then copies each into a contiguous [NB][L][d] buffer before the call (models/attention_blockcuda.py:48,80;
 * the output is copied back by combine_heads, models/attention.py:131-134).  These two entry points read and
 * write such views in place.  Element (b, h, i, f) of a tensor lies batch_stride*b + head_stride*h +
 * row_stride*i + f floats after its pointer; one layout for the inputs Q, K, V, one for Out and dO, one for
 * the gradients dQ, dK, dV.  heads = H (num_batches of the handle = B*H, head index fastest).  Strides are
 * multiples of 4 floats, pointers 16-byte aligned, seq_len * row_stride < 2^29; the layouts of tensors that are
 * written (out, grad) must not map two elements to one address, those of inputs may (head_stride 0: one K / V
 * head shared by all query heads).  Served by every kernel family: the tile kernels (emb_dim 32 or 64, patterns
 * of aligned 32x32 tiles), the hybrid kernels (emb_dim 32) and the element kernels (emb_dim 16, 32, 64, 128);
 * the results equal those of the row-major entry points bit for bit.  Attn / P stay [NB][nnz] as everywhere.
 * The kept copies of Out are not used: the backward takes Out (required).  On patterns without tile structure
 * the backward's dS scratch ([NB][nnz] floats) belongs to the handle and is allocated by the first such call
 * (not under HIP graph capture).  Workspaces that follow the pattern's size grow when a larger pattern arrives; the
 * buffer a larger one replaces stays allocated until the handle is destroyed, so a HIP graph recorded earlier on
 * the handle can still be replayed. */
typedef struct spion_head_layout {
    long long batch_stride;
    int head_stride;
    int row_stride;
} spion_head_layout;
void spion_attn_forward_strided(void* handle, const float* Q, const float* K, const float* V, const float* Mask,
                                float* Attn, float* Out,
                                const int* Offsets, const int* Columns, const int* SumMat, int nnz,
                                int heads, const spion_head_layout* in, const spion_head_layout* out);
void spion_attn_backward_strided(void* handle, const float* Q, const float* K, const float* V, const float* P,
                                 const float* Out, const float* dO,
                                 float* dQ, float* dK, float* dV,
                                 const int* Offsets, const int* Columns, const int* SumMat, int nnz,
                                 int heads, const spion_head_layout* in, const spion_head_layout* out,
                                 const spion_head_layout* grad);

/* The bf16 family on the same kind of views (no counterpart in the reference; models/attention.py:136-139 is where
 * its fp32 layer makes them): Q, K, V / Out, dO / dQ, dK, dV as [B][H][L][d] views located by one layout per group,
 * strides in bf16 elements and multiples of 8, pointers 16-byte aligned; Lse and Mask stay [NB][L].  Same kernels
 * and arithmetic as the contiguous entry points: bit-identical results. */
void spion_block_bf16_attn_forward_strided(void* handle, const void* Q, const void* K, const void* V, const float* Mask,
                                           void* Out, float* Lse,
                                           const int* Offsets, const int* Columns, const int* SumMat, int nnz,
                                           int heads, const spion_head_layout* in, const spion_head_layout* out);
void spion_block_bf16_attn_backward_strided(void* handle, const void* Q, const void* K, const void* V, const float* Mask,
                                            const void* Out, const float* Lse, const void* dO,
                                            void* dQ, void* dK, void* dV,
                                            const int* Offsets, const int* Columns, const int* SumMat, int nnz,
                                            int heads, const spion_head_layout* in, const spion_head_layout* out,
                                            const spion_head_layout* grad);

/* The dense phase on the same views: the reference's dense modules transpose Q and V before the forward and K
 * and grad_output before the backward (models/attention_cuda.py:22-31,52-62) because its GEMM calls
 * (models/attn.cu:179-262) take feature-major operands, and hand Out and the gradients back feature-major.
 * Here Q, K, V, Out, dO, dQ, dK, dV are all [B][H][L][d] views described as above (a contiguous [NB][L][d]
 * tensor is the layout {H*L*d, L*d, d}); Attn / P is the same [NB][key][query] map as in attn_forward.  Mask:
 * NULL for a handle of spion_dense_init, the [NB][L] penalty for one of spion_densemask_init.  seq_len <= 16384;
 * with emb_dim 64 the forward serves seq_len <= 2048 (the backward all of them).  No copy of Out is kept: the
 * backward takes Out (required). */
void spion_dense_forward_strided(void* handle, const float* Q, const float* K, const float* V, const float* Mask,
                                 float* Attn, float* Out,
                                 int heads, const spion_head_layout* in, const spion_head_layout* out);
void spion_dense_backward_strided(void* handle, const float* Q, const float* K, const float* V, const float* P,
                                  const float* Out, const float* dO,
                                  float* dQ, float* dK, float* dV,
                                  int heads, const spion_head_layout* in, const spion_head_layout* out,
                                  const spion_head_layout* grad);

/* The dense forward on [B][H][L][d] views (spion_dense_forward_strided) that also leaves the mean of all
 * num_batches maps in Mean [seq_len][seq_len] (queries x keys, the Score input of spion_pattern_generate):
 * models/model_transformer.py:136-137 takes that mean with two torch.mean passes over the [B,H,L,L] tensor the
 * forward has just written; here every map tile is added to a partial sum while it is on its way to memory, and
 * one reduction over a few partial maps finishes the mean, so the maps are not read back.  The handle keeps the
 * partial maps: C * seq_len^2 floats, C = the smallest divisor of num_batches with C * seq_len / 32 >= 512, or
 * num_batches itself when it has none; allocated by the first such call (not under HIP graph capture).  All other arguments and results as in
 * spion_dense_forward_strided (Attn is still written: the API returns it).  emb_dim 32 only. */
void spion_dense_forward_strided_mean(void* handle, const float* Q, const float* K, const float* V, const float* Mask,
                                      float* Attn, float* Out, float* Mean,
                                      int heads, const spion_head_layout* in, const spion_head_layout* out);

/* Host-side helper: out[b][c][r] = in[b][r][c] (fp32), for the transposed K / V / Q / dO operands the
 * attention entry points take.  Returns 0 on success. */
int spion_transpose_last2(const float* in, float* out, int batch, int rows, int cols, void* stream);

const char* spion_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SPION_HIP_H */
