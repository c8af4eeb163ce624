/* clgrpo.h - C ABI of the MI355X (gfx950) GRPO/GSPO policy-loss library.
 *
 * Plain C, no torch types.  Every tensor argument is a caller-owned pointer;
 * device pointers unless the comment says "host".  Launching entry points take
 * a hipStream_t (passed as void*) and only enqueue work on it.  They never
 * allocate: scratch memory comes in through `workspace`, whose size the
 * matching *_workspace_bytes() function reports.  Return value: 0, or a
 * negative clgrpo_status; clgrpo_last_error_string() gives the reason for the
 * calling thread.
 *
 * The reference (alibaba/ChatLearn) has no FFI: the functions named beside each
 * entry point are the Python functions whose arithmetic the entry point
 * replaces, paths relative to chatlearn/algorithm/grpo_utils/.
 */
#ifndef CLGRPO_H_
#define CLGRPO_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  CLGRPO_OK = 0,
  CLGRPO_EINVAL = -1,     /* bad scalar argument (negative size, bad mode, ...) */
  CLGRPO_EDTYPE = -2,     /* unsupported dtype enum */
  CLGRPO_ESHAPE = -3,     /* shape the kernels cannot take (e.g. H not a multiple of 64) */
  CLGRPO_ENULL = -4,      /* required pointer is NULL */
  CLGRPO_ELAUNCH = -5,    /* HIP reported an error at launch */
  CLGRPO_EWORKSPACE = -6  /* workspace too small */
} clgrpo_status;

typedef enum { CLGRPO_BF16 = 0, CLGRPO_F32 = 1, CLGRPO_F64 = 2, CLGRPO_U8 = 3 /* bool / uint8 flags */ } clgrpo_dtype;

/* major * 100 + minor.  A change of an args struct's layout or of a buffer's meaning raises the major part;
 * callers compare clgrpo_version() / 100 with the CLGRPO_VERSION / 100 they were built against.
 *   1.00 -> 2.00: clgrpo_lmhead_fwd_args / clgrpo_lmhead_bwd_args gained saved_rows (must be set whenever
 *                 saved_logits is); clgrpo_softmax_stats_bwd_args gained lse and entropy; kept logits of 16-bit
 *                 inputs are IEEE half in the forward's own order; clgrpo_lmhead_fwd_workspace_bytes grew to
 *                 min(ceil(V / 256), 64) * T * 16.
 *   2.00 -> 2.01: clgrpo_lmhead_bwd_workspace_bytes sizes the split-K partials by the GEMM's plan (smaller in
 *                 general); clgrpo_lmhead_fwd_launch_plan and clgrpo_lmhead_bwd_dhidden_plan added.
 *   2.01 -> 2.02: clgrpo_lmhead_bwd_workspace_bytes also covers the partials of the dW GEMM's tail launch (a few
 *                 tens of MB more for some shapes); clgrpo_lmhead_bwd_dweight_plan added. */
#define CLGRPO_VERSION 202
int clgrpo_version(void);
const char* clgrpo_last_error_string(void);

/* ------------------------------------------------------------------ *
 * Fused lm_head projection + online log-softmax statistics.
 * Replaces: model(...).logits (policy_trainer.py:216-221, nn.Linear(H,V)),
 * logprobs_from_logits (trainer_utils.py:46-52), entropy_from_logits[_with_chunking]
 * (trainer_utils.py:27-44), Megatron CE + _VocabParallelEntropy at tp=1
 * (megatron_utils/train_helper.py:480-482,605-627).  The [T,V] logits are never
 * written to memory.
 * ------------------------------------------------------------------ */
typedef struct {
  const void* hidden;      /* [T, H] row-major, `dtype` */
  const void* weight;      /* [V, H] row-major, `dtype` (lm_head.weight) */
  const int64_t* labels;   /* [T]; NULL => logprob is not produced */
  int64_t T, H, V;
  int32_t dtype;           /* CLGRPO_BF16 or CLGRPO_F32 */
  float inv_temperature;   /* logits are multiplied by this before the softmax (1/tau) */
  float* logprob;          /* [T] out, fp32; may be NULL iff labels is NULL */
  float* entropy;          /* [T] out, fp32; may be NULL */
  float* rowmax;           /* [T] out, fp32 (max_v z); may be NULL */
  float* lse;              /* [T] out, fp32 (logsumexp_v z); required */
  void* workspace;
  size_t workspace_bytes;
  void* saved_logits;      /* optional out: the raw logits hidden.W^T (before the temperature), for a later
                              clgrpo_lmhead_bwd of the SAME rows that then skips the recomputation.  NULL: nothing
                              is stored.  Callers bound its size by processing a micro-batch in token chunks.
                              The buffer is opaque to the caller: ceil(rows / 256) * 256 rows of ld_saved elements
                              of sizeof(dtype) bytes.  The forward fills it in the order of its accumulators
                              (32 KB units of 256 rows x 128 bytes of vocabulary, inside a unit 32 x 32 sub-blocks
                              stored as 16-byte pieces per lane; 16-bit inputs keep their logits as IEEE half, a raw
                              logit beyond +-65504 as +-65504: the backward's gradients stay finite, but that
                              token's probabilities are then formed from the saturated value);
                              the backward overwrites every unit in place with d(logits) as the K-blocked operand
                              of its GEMMs: element (row, k) at
                              (((row / 256) * (ld_saved / E) + k / E) * 256 + row % 256) * E + k % E,
                              E = 128 / sizeof(dtype). */
  int64_t ld_saved;        /* K extent in elements, a multiple of 64, >= clgrpo_saved_logits_ld(V) */
  const int32_t* saved_row_map; /* optional [T]: row of saved_logits that receives token t's logits, or a
                              negative value to store nothing for t (tokens whose upstream gradient is
                              known to be zero, e.g. masked-out prompt positions).  NULL: row t. */
  int64_t saved_rows;      /* rows the buffer can address (a multiple of 256 is allocated; see above); a
                              mapped row outside [0, saved_rows) is not stored */
} clgrpo_lmhead_fwd_args;

/* Row stride (elements) the saved-logits buffer must have: V rounded up to 64. */
int64_t clgrpo_saved_logits_ld(int64_t V);

size_t clgrpo_lmhead_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int32_t dtype);
int clgrpo_lmhead_fwd(const clgrpo_lmhead_fwd_args* a, void* stream);
/* The grid of the forward launch for T tokens on a device with `cus` compute units (<= 0: 256):
 * out[0] = blocks of 256 tokens, out[1] = vocabulary splits (a workgroup owns one token block and one split),
 * out[2] = vocabulary tiles of 256 entries a workgroup walks.  The launch takes ceil(out[0] * out[1] / cus)
 * rounds of one workgroup per compute unit.  Host-side arithmetic only; no counterpart in the reference
 * (its lm_head is one library GEMM). */
int clgrpo_lmhead_fwd_launch_plan(int64_t T, int64_t V, int32_t cus, int32_t* out);

/* ------------------------------------------------------------------ *
 * Backward of the fused head: recomputes logit tiles from hidden, W and the
 * stored lse, forms d(logits) and contracts it into dhidden and dW.
 * Replaces: autograd through lm_head / log_softmax / entropy at
 * policy_trainer.py:286 (total_loss.backward()).
 *   dz[t,v] = g_logprob[t] (1[v==label_t] - p[t,v]) - g_entropy[t] p[t,v] (log p[t,v] + entropy[t])
 *   dhidden = inv_temperature * dz W        dW (+)= inv_temperature * dz^T hidden
 * ------------------------------------------------------------------ */
typedef struct {
  const void* hidden;       /* [T, H] `dtype` */
  const void* weight;       /* [V, H] `dtype` */
  const int64_t* labels;    /* [T] */
  const float* lse;         /* [T] from the forward */
  const float* entropy;     /* [T] from the forward; required iff g_entropy != NULL */
  const float* g_logprob;   /* [T] upstream gradient of logprob */
  const float* g_entropy;   /* [T] upstream gradient of entropy, or NULL */
  int64_t T, H, V;
  int32_t dtype;
  float inv_temperature;
  void* dhidden;            /* [T, H] out, `dtype`; NULL => skipped */
  float* dweight;           /* [V, H] out, fp32; NULL => skipped */
  int32_t accumulate_dweight; /* nonzero: dweight += ; zero: dweight = */
  void* workspace;
  size_t workspace_bytes;   /* sets the token chunk: see clgrpo_lmhead_bwd_workspace_bytes */
  void* saved_logits;       /* optional in/out: logits stored by clgrpo_lmhead_fwd for these rows (the same opaque
                               buffer, ceil(T / 256) * 256 rows of ld_saved elements).  Overwritten in place
                               with d(logits); the recomputation is skipped. */
  int64_t ld_saved;
  void* weight_t;           /* optional, `dtype`: caller-kept W^T in the same blocked layout (ceil(H / 256) * 256
                               rows of clgrpo_saved_logits_ld(V) elements), so that several calls with the same
                               weight (token chunks of one step) build it once */
  int32_t weight_t_ready;   /* zero: this call fills weight_t; nonzero: it already holds W^T */
  int64_t saved_rows;       /* rows the saved_logits buffer holds; must be >= ceil(T / 256) * 256 (the backward
                               rewrites whole 256-row units) */
} clgrpo_lmhead_bwd_args;

/* Bytes needed to process `chunk_tokens` tokens at a time (chunk_tokens <= 0: all T at once).
 * with_saved_logits is a bit set: bit 0: the d(logits) buffer is the caller's saved_logits, not part of the
 * workspace; bit 1: the caller keeps W^T (weight_t), so the workspace holds no copy of it. */
size_t clgrpo_lmhead_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int32_t dtype,
                                         int64_t chunk_tokens, int32_t with_saved_logits);
int clgrpo_lmhead_bwd(const clgrpo_lmhead_bwd_args* a, void* stream);
/* How the dhidden contraction of `rows` tokens is launched on a device with `cus` compute units (<= 0: 256):
 * out[0] = 256-token tiles of a first launch that fills whole rounds without cutting K (0: one launch over
 * all rows), out[1] = K ranges of the (remaining) launch, whose fp32 partial tiles a second pass sums.
 * Host-side arithmetic only; no counterpart in the reference. */
int clgrpo_lmhead_bwd_dhidden_plan(int64_t rows, int64_t H, int64_t V, int32_t dtype, int32_t cus, int32_t* out);
/* How the dW contraction over a chunk of `rows` tokens is launched: out[0] = walks (workgroups that keep one
 * 256-column tile of hidden^T and walk runs of vocabulary tiles; 0: one workgroup per tile), out[1] = vocabulary
 * tiles of a first launch whose walks are all equally long (0: one launch over all of them), out[2] = K ranges of
 * the launch over the remaining vocabulary tiles (fp32 partial tiles, summed by a second pass).
 * Host-side arithmetic only; no counterpart in the reference. */
int clgrpo_lmhead_bwd_dweight_plan(int64_t rows, int64_t H, int64_t V, int32_t dtype, int32_t cus, int32_t* out);

/* ------------------------------------------------------------------ *
 * One vocabulary shard of the head (tensor-parallel lm_head: each rank keeps rows
 * [vocab_begin, vocab_begin + V) of the weight).  Replaces, per rank, the local part of
 * Megatron's vocab-parallel cross entropy and of _VocabParallelEntropy
 * (megatron_utils/train_helper.py:605-627): instead of three all-reduces over [T] (max,
 * sum of exponentials, sum of p*z) plus the target-logit reduce, a rank produces one 16-byte
 * record per token; the records of all ranks (exchanged by the caller) are merged exactly.
 *
 *   record[t] = (max_v z, sum_v 2^((z-max)*c), sum_v 2^((z-max)*c) * z, z[label] if the label
 *                falls in this shard else 0),   z = raw shard logits, c = log2(e) * inv_temperature
 *
 * clgrpo_lmhead_fwd_shard: `a` as for clgrpo_lmhead_fwd with V = rows of this shard and GLOBAL label
 * ids; a->logprob / entropy / rowmax / lse are ignored (may be NULL); saved_logits keeps the shard's
 * logits as usual.  clgrpo_lmhead_merge_shards: records laid out [n_shards][T]; V_total bounds the
 * labels (outside => NaN logprob).  clgrpo_lmhead_bwd_shard: `a` as for clgrpo_lmhead_bwd with the
 * shard's weight and V, GLOBAL labels, and the merged lse / entropy; dweight is the shard's rows,
 * dhidden this shard's partial sum (the caller adds the shards').
 * ------------------------------------------------------------------ */
int clgrpo_lmhead_fwd_shard(const clgrpo_lmhead_fwd_args* a, int64_t vocab_begin, void* record /* float4 [T] */,
                            void* stream);
int clgrpo_lmhead_merge_shards(const void* records, int64_t n_shards, int64_t T, const int64_t* labels,
                               int64_t V_total, float inv_temperature, float* logprob, float* entropy,
                               float* rowmax, float* lse, void* stream);
int clgrpo_lmhead_bwd_shard(const clgrpo_lmhead_bwd_args* a, int64_t vocab_begin, void* stream);

/* ------------------------------------------------------------------ *
 * Softmax statistics from materialised logits (legacy call sites that already
 * hold [R, V] logits) and the matching backward.
 * Replaces: logprobs_from_logits, entropy_from_logits, entropy_from_logits_with_chunking,
 * entropy_from_tensor_parallel_logits (tp=1).
 * ------------------------------------------------------------------ */
typedef struct {
  const void* logits;      /* [R, V] row-major with row stride `ld` elements */
  const int64_t* labels;   /* [R] or NULL */
  int64_t R, V, ld;
  int32_t dtype;           /* CLGRPO_BF16 or CLGRPO_F32 */
  float* logprob;          /* [R] or NULL */
  float* entropy;          /* [R] or NULL */
  float* lse;              /* [R] or NULL */
} clgrpo_softmax_stats_args;
int clgrpo_softmax_stats(const clgrpo_softmax_stats_args* a, void* stream);

typedef struct {
  const void* logits;      /* [R, V] */
  const int64_t* labels;   /* [R] or NULL (required iff g_logprob) */
  const float* g_logprob;  /* [R] or NULL */
  const float* g_entropy;  /* [R] or NULL */
  int64_t R, V, ld;
  int32_t dtype;
  void* dlogits;           /* [R, V] out, `dtype`, row stride V */
  const float* lse;        /* [R] from clgrpo_softmax_stats, or NULL: the row statistics are then rebuilt by one
                              more pass over the logits */
  const float* entropy;    /* [R] from clgrpo_softmax_stats; used (with lse) when g_entropy != NULL */
} clgrpo_softmax_stats_bwd_args;
int clgrpo_softmax_stats_bwd(const clgrpo_softmax_stats_bwd_args* a, void* stream);

/* ------------------------------------------------------------------ *
 * Clipped importance-ratio policy loss (token-level GRPO or sequence-level
 * GSPO), k3 KL estimator, masked sums and the per-token upstream gradients.
 * Replaces: calculate_grpo_loss (loss_gallery.py:6-33), calculate_gspo_loss
 * (loss_gallery.py:35-74), the loss assembly of policy_trainer.py:263-286 and
 * _compute_all_losses / loss_func of megatron_utils/train_helper.py:426-547.
 *
 * Tokens are addressed flat, n = total elements.  Sequence of token i:
 *   cu_seqlens != NULL : packed, the b with cu_seqlens[b] <= i < cu_seqlens[b+1]
 *   cu_seqlens == NULL : padded [B, S] row-major, b = i / S.
 * ------------------------------------------------------------------ */
typedef enum { CLGRPO_LOSS_GRPO = 0, CLGRPO_LOSS_GSPO = 1 } clgrpo_loss_mode;

typedef struct {
  int32_t mode;              /* clgrpo_loss_mode */
  int32_t compute_dtype;     /* CLGRPO_F32 or CLGRPO_F64: type of advantages, loss, dloss */
  int64_t n;                 /* tokens */
  int64_t B;                 /* sequences */
  int64_t S;                 /* padded row length (used iff cu_seqlens == NULL) */
  const int32_t* cu_seqlens; /* [B+1] or NULL */
  const float* logprob;      /* [n] */
  const float* old_logprob;  /* [n] */
  const float* ref_logprob;  /* [n] or NULL (no KL term) */
  const float* entropy;      /* [n] or NULL */
  const int32_t* loss_mask;  /* [n] or NULL (= all ones) */
  const void* advantages;    /* [B] compute_dtype */
  double diff_clip_ratio, pos_clip_ratio, neg_clip_ratio, final_clip_ratio;
  double kl_coef, entropy_coef; /* used only for g_logprob / g_entropy */
  double grad_scale;         /* fsdp_size / N of policy_trainer.py:266-285 */
  void* loss;                /* [n] out compute_dtype: per-token surrogate (unmasked) */
  void* dloss_dlogprob;      /* [n] out compute_dtype or NULL: d loss[i] / d logprob[i] */
  float* kl;                 /* [n] out fp32 or NULL: clamp(exp(k)-k-1,-10,10), k=ref-lp,
                                with exp(k) replaced by 1 where the mask is 0 (train_helper.py:524) */
  uint8_t* is_positive_clipped; /* [n] or NULL (GSPO flags; also defined for GRPO) */
  uint8_t* is_negative_clipped; /* [n] or NULL */
  uint8_t* is_clipped;          /* [n] or NULL */
  float* g_logprob;          /* [n] out or NULL: mask*grad_scale*(dloss + kl_coef*dkl) */
  float* g_entropy;          /* [n] out or NULL: -entropy_coef*mask*grad_scale */
  double* sums;              /* [8] out: sum(mask*loss), sum(mask*kl), sum(mask*entropy), sum(mask),
                                sum(mask*pos), sum(mask*neg), sum(mask*clipped), 0 */
  int32_t* flags;            /* [1] out: bit0 loss has NaN, bit1 exp(k) has Inf, bit2 exp(k) has NaN */
  void* workspace;
  size_t workspace_bytes;
  int64_t token_offset;      /* packed layout: position of token 0 of this call inside the row that
                                cu_seqlens describes (lets a caller walk a micro-batch in token chunks) */
} clgrpo_policy_loss_args;

size_t clgrpo_policy_loss_workspace_bytes(int64_t n, int64_t B);
int clgrpo_policy_loss(const clgrpo_policy_loss_args* a, void* stream);
/* Kernel launches one clgrpo_policy_loss call of n tokens enqueues: 1 up to 4096 tokens (sequence means,
 * per-token pass, sums and flag word in a single workgroup), else 2 (per-token pass, finalize) plus 1 for
 * the sequence means of CLGRPO_LOSS_GSPO. */
int clgrpo_policy_loss_launches(int64_t n, int32_t mode);

/* clgrpo_policy_loss without a workspace and without any allocation.  No counterpart in the reference: it
 * is for callers that cannot allocate device memory around the call (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  Same arguments and results as clgrpo_policy_loss,
 * bit for bit; `workspace` / `workspace_bytes` are ignored (may be NULL / 0).  The scratch memory is a
 * 320 KiB array built into the library, one copy per device: at most
 * clgrpo_policy_loss_static_max_sequences() = 65536 sequences per call (any number of tokens), more is
 * refused with CLGRPO_EWORKSPACE.  Calls that overlap on one device (two streams) share the array and race:
 * keep them in stream order, or use clgrpo_policy_loss with separate workspaces. */
int clgrpo_policy_loss_static(const clgrpo_policy_loss_args* a, void* stream);
int64_t clgrpo_policy_loss_static_max_sequences(void);

/* Masked reductions of a dict of per-token loss tensors, one launch.
 * Replaces: the body of loss_func (megatron_utils/train_helper.py:441-463):
 *   out[j] = sum_i float(src_j[i]) * mask[i]                       (average[j] == 0)
 *   out[j] = sum_i float(src_j[i]) * mask[i] / (1e-5 + sum(mask))  (average[j] != 0, the *_sample_average keys)
 *   count  = sum(mask)
 * and, for the one key that is back-propagated (pg_loss), its gradient mask * g. */
typedef struct {
  int64_t n;                 /* elements per tensor */
  int32_t k;                 /* tensors, 1..16 */
  const void* src[16];       /* [n] each */
  int32_t dtype[16];         /* CLGRPO_F32, CLGRPO_F64 or CLGRPO_U8 (bool flags) */
  int32_t average[16];
  const int32_t* mask;       /* [n] */
  float* out;                /* [k] out */
  int32_t* count;            /* [1] out */
} clgrpo_masked_sums_args;
int clgrpo_masked_sums(const clgrpo_masked_sums_args* a, void* stream);
/* dst[i] = g[0] * mask[i] in `dtype` (CLGRPO_F32 / CLGRPO_F64); g is a device scalar. */
int clgrpo_masked_sums_bwd(int64_t n, const float* g, const int32_t* mask, void* dst, int32_t dtype, void* stream);

/* ------------------------------------------------------------------ *
 * Group-wise reward -> advantage: adv = (r - mean(pool_g)) / (std(pool_g) + eps),
 * population std, float64.  Replaces: AdvantageComputer.__call__ arithmetic
 * (advantage_compute.py:27-36).  pool holds, group after group, every reward
 * buffered for that prompt (this call's and carried-over ones).
 * ------------------------------------------------------------------ */
typedef struct {
  int64_t n_samples, n_groups;
  const double* rewards;      /* [n_samples] */
  const int32_t* group_of;    /* [n_samples] group index of each sample */
  const double* pool;         /* [pool_offsets[n_groups]] */
  const int32_t* pool_offsets;/* [n_groups+1] */
  double eps;
  double* advantages;         /* [n_samples] out */
  uint8_t* all_zeros;         /* [n_samples] out: every pooled reward of the group == 0 */
  uint8_t* all_ones;          /* [n_samples] out: every pooled reward of the group == 1 */
} clgrpo_group_advantage_args;
int clgrpo_group_advantage(const clgrpo_group_advantage_args* a, void* stream);

/* ------------------------------------------------------------------ *
 * Mask / index builders for padded <-> packed batches (bit-exact integers).
 * Replaces: generate_loss_mask_position_ids (trainer_utils.py:60-96, text branch),
 * the label roll and training-mask shift (policy_trainer.py:135,160-162;
 * train_helper.py:405-413), unpad_input (trainer_utils.py:155-194) and the
 * flash-attn index_first_axis / pad_input it relies on.
 * ------------------------------------------------------------------ */
typedef struct {
  int64_t B, S;
  const int32_t* prompt_len;   /* [B] */
  const int32_t* response_len; /* [B] */
  int32_t* attn_mask;          /* [B,S] out */
  int32_t* loss_mask;          /* [B,S] out */
  int64_t* position_ids;       /* [B,S] out or NULL */
} clgrpo_build_masks_args;
int clgrpo_build_masks(const clgrpo_build_masks_args* a, void* stream);

typedef struct {
  int64_t B, S;
  const int64_t* tokens;       /* [B,S] or NULL */
  const int32_t* loss_mask;    /* [B,S] or NULL */
  int64_t* labels;             /* [B,S] out: tokens rolled left by one along S (wraps) */
  int32_t* shifted_mask;       /* [B,S] out: mask rolled left by one along S */
  int32_t zero_last;           /* nonzero: shifted_mask[:, S-1] = 0 (FSDP trainer) */
} clgrpo_shift_labels_args;
int clgrpo_shift_labels(const clgrpo_shift_labels_args* a, void* stream);

typedef struct {
  int64_t B, S;
  const int32_t* attn_mask;    /* [B,S] */
  int64_t* indices;            /* [B*S] out: flat positions of the nonzero mask entries, ascending;
                                  only the first total[0] are written */
  int32_t* cu_seqlens;         /* [B+1] out */
  int32_t* seqlens;            /* [B] out */
  int32_t* total;              /* [2] out: {number of indices written, max seqlen} */
  int32_t* row_offsets;        /* [B+1] scratch */
} clgrpo_unpad_indices_args;
int clgrpo_unpad_indices(const clgrpo_unpad_indices_args* a, void* stream);

/* Packed ("THD") micro-batch for the Megatron trainer in one pass, driven by the per-sample
 * (prompt, response) lengths.  Replaces the packed branch of get_batch
 * (megatron_utils/train_helper.py:258-328): the O(B) Python loops that build the attention mask,
 * pad every sequence to a multiple of align = tp*cp*2 with the eod token, unpad_input, the label
 * roll, the loss mask placed at cu_seqlens_padded[i] + prompt and rolled, and
 * thd_get_partitioned_indices (TransformerEngine) with the index_select calls that follow it.
 *
 * Row i of the padded batch holds seqlen_i = prompt_i + response_i tokens; its packed segment has
 * padded_i = ceil(seqlen_i / align) * align tokens.  The caller passes total_padded = sum padded_i
 * (known on the host from the same lengths); the call fails the `status` word (bit 0) if the device
 * sum disagrees, (bit 1) if a sequence is longer than S, (bit 2) if cp_size > 1 and a padded length is
 * not a multiple of 2*cp_size.
 * Outputs over the whole packed row (n = total_padded):
 *   cu_seqlens_padded [B+1], seqlens [B], seqlens_padded [B]            int32
 *   stats[0] = total_padded, stats[1] = max padded length                int32
 *   indices [n]: position in the padded [B, max padded length] layout    int64
 * Outputs for this context-parallel rank (m = total_padded / cp_size entries, order of seq_indices):
 *   seq_indices [m]: positions in the packed row this rank owns (per sequence the chunks
 *                    cp_rank and 2*cp_size-1-cp_rank of 2*cp_size equal chunks)        int64
 *   tokens [m], labels [m] (packed row rolled left by one, wrapping)    int64
 *   loss_mask [m] (rolled the same way)                                  int32
 *   stats[2] = number of ones in loss_mask                               int32
 * With align = 1 and cp_size = 1 this is also the packing step of the FSDP trainer (unpad_input of the
 * tokens and position ids plus the label roll, policy_trainer.py:143-162) without its host round trip.
 */
typedef struct {
  int64_t B, S;
  const int64_t* tokens;        /* [B,S] */
  const int32_t* prompt_len;    /* [B] */
  const int32_t* response_len;  /* [B] */
  int32_t align;                /* tp*cp*2 */
  int32_t cp_size, cp_rank;
  int64_t pad_token;            /* tokenizer eod */
  int64_t total_padded;
  int32_t* cu_seqlens_padded;   /* [B+1] out */
  int32_t* seqlens;             /* [B] out */
  int32_t* seqlens_padded;      /* [B] out */
  int32_t* stats;               /* [3] out */
  int32_t* status;              /* [1] out, zero when consistent */
  int64_t* indices;             /* [total_padded] out */
  int64_t* seq_indices;         /* [total_padded / cp_size] out */
  int64_t* out_tokens;          /* [total_padded / cp_size] out */
  int64_t* out_labels;          /* [total_padded / cp_size] out */
  int32_t* out_loss_mask;       /* [total_padded / cp_size] out, or NULL */
  int64_t* out_position_ids;    /* [total_padded / cp_size] out, or NULL: position of the token inside its sequence
                                   (what unpad_input gives for the padded arange position ids, policy_trainer.py:152-156) */
} clgrpo_thd_pack_args;
int clgrpo_thd_pack(const clgrpo_thd_pack_args* a, void* stream);

typedef struct {
  const void* src;             /* gather: [n_src_rows, row_bytes]; scatter: [n_idx, row_bytes] */
  void* dst;                   /* gather: [n_idx, row_bytes];      scatter: [n_dst_rows, row_bytes] */
  const int64_t* indices;      /* [n_idx] */
  int64_t n_idx, row_bytes;
  int64_t n_rows;              /* rows of the indexed side (bounds check on the host is the caller's) */
} clgrpo_rows_args;
int clgrpo_gather_rows(const clgrpo_rows_args* a, void* stream);   /* dst[i] = src[indices[i]] */
int clgrpo_scatter_rows(const clgrpo_rows_args* a, void* stream);  /* dst = 0; dst[indices[i]] = src[i] */

/* ------------------------------------------------------------------ *
 * Host-side bin packing for dynamic batching (runs on the CPU, like the
 * reference's).  Replaces: bin_packing (packing_utils.py:23-54) and
 * bin_packing_fix_bin (packing_utils.py:56-83).  All pointers are HOST memory.
 * bin_of[i] receives the bin of item i; order[] receives the item ids bin after
 * bin in insertion order, bin_offsets[b]..bin_offsets[b+1] delimiting bin b.
 * ------------------------------------------------------------------ */
int clgrpo_bin_packing(const int64_t* seq_len, int64_t n, int64_t max_train_token,
                       int64_t* order, int64_t* bin_offsets, int64_t* n_bins);
int clgrpo_bin_packing_fix_bin(const int64_t* seq_len, int64_t n, int64_t bin_size,
                               int64_t* order, int64_t* bin_offsets);

#ifdef __cplusplus
}
#endif
#endif /* CLGRPO_H_ */
