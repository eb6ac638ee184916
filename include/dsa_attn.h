/*
 * dsa_attn.h - C ABI of the MI355X (gfx950) packed-sequence DSA attention library.
 *
 * The library replaces the one device routine the reference's attention layers call,
 *   torch.nn.attention.varlen.varlen_attn(q, k, v, cu_seq_q, cu_seq_k, max_q, max_k, window_size=(-1, 0))
 * reached from train/model_attention.py:123-132, models/qwen3_vl/model.py:41-46 and
 * models/qwen3_5/model.py:93-98, and extends it with the four DSA stages
 * (indexer score -> top-k -> sparse forward -> sparse backward).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless it says "host"; tensors are row-major contiguous;
 *   - q (T,Hq,D), k/v (T,Hkv,D), q_idx (T,Hi,Di), k_idx (T,Di), w_idx (T,Hi): bf16 (dtype code below);
 *   - cu_seqlens (N+1) int32, cu[0]=0, cu[N]=T, non-decreasing (zero-length segments allowed, the pad
 *     tail is one more segment: data/energon_dataloader.py:431-464, models/qwen3_vl/model.py:757-765);
 *   - idx (T,K) int32: global packed row ids of the selected keys, ascending, padded with -1;
 *     n (T) int32: how many are valid.  idx == NULL and n == NULL select every causal key of the
 *     token's own segment (the reference's dense causal semantics);
 *   - lse (Hq,T) fp32 natural-log softmax normaliser (what the flash kernel behind varlen_attn saves);
 *   - stream is a hipStream_t passed as void*; all work is ordered on it, nothing synchronises (the backward may run
 *     one of its passes on a second stream between a fork and a join event on this one: dsa_set_bwd_overlap);
 *   - every entry returns 0 on success or a negative dsa_status; dsa_last_error() gives the text
 *     (thread-local).  No exception crosses the boundary.
 */
#ifndef DSA_ATTN_H
#define DSA_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    DSA_OK = 0,
    DSA_ERR_ARG = -1,          /* bad shape / null pointer / inconsistent sizes */
    DSA_ERR_UNSUPPORTED = -2,  /* dtype or head geometry the kernels do not cover */
    DSA_ERR_WORKSPACE = -3,    /* workspace too small */
    DSA_ERR_HIP = -4           /* a HIP call or launch failed */
} dsa_status;

#define DSA_DTYPE_BF16 0
#define DSA_DTYPE_FP32 1 /* accepted by the Python host only (it rounds to bf16 first) */

/* Library identification, e.g. "dsa-attn-gfx950 0.1".  (no reference counterpart) */
const char *dsa_version(void);
/* Text of the last error raised on the calling thread ("" if none). */
const char *dsa_last_error(void);

/*
 * Stage D1 - lightning-indexer scores for the query rows [row_begin,row_end).
 *   scores[(t-row_begin)*ld + (s - seg_start(t))] = scale * sum_j w[t,j] * relu(q_idx[t,j,:] . k_idx[s,:])
 * for s in [seg_start(t), t].  Columns beyond the row's own position are left untouched.
 * Rows with pos(t)+1 <= skip_dense_k are skipped (their top-k is the whole causal window).
 * No reference counterpart (the reference has no indexer); formula of the DSA operator.
 */
int dsa_indexer_scores(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu_seqlens,
                       int T, int N, int Hi, int Di, float scale, int dtype, int row_begin, int row_end,
                       int skip_dense_k, float *scores, int64_t ld, void *stream);

/*
 * Stage D2 - per-query top-k of materialised scores (also the bit-exactness test hook).
 * Row t keeps the min(K, pos+1) columns first under (score descending, column ascending); -0.0 == +0.0.
 * Writes global row ids ascending into idx[t*K ...], -1 padded, and n[t].
 */
int dsa_topk_from_scores(const float *scores, int64_t ld, int row_begin, int row_end, const int32_t *cu_seqlens,
                         int T, int N, int K, int32_t *idx, int32_t *n, void *stream);

/* Bytes of workspace dsa_index_topk needs (score rows are produced in chunks that fit). */
size_t dsa_index_topk_workspace_bytes(int T, int max_seqlen, int K);

/*
 * Stages D1+D2 over the whole packed batch.  ws must hold dsa_index_topk_workspace_bytes().
 * Stands where a DSA layer would call its indexer before attention; no reference counterpart.
 */
int dsa_index_topk(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu_seqlens,
                   int T, int N, int Hi, int Di, int K, float scale, int dtype, int max_seqlen,
                   int32_t *idx, int32_t *n, void *ws, size_t ws_bytes, void *stream);

/*
 * dsa_index_topk for callers that cannot allocate device memory or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same arguments without `ws`, same idx and n, bit
 * for bit.  It has no counterpart in the reference.  The score rows are kept in a static device array of
 * dsa_index_topk_noalloc_scratch_bytes() = 32 MiB that every GPU the library runs on holds until the process ends;
 * the rows are worked through in chunks that fit, so T is unlimited and only max_seqlen is bounded:
 * max_seqlen > dsa_index_topk_noalloc_max_seqlen() (2 097 152) returns DSA_ERR_WORKSPACE.  The call allocates
 * nothing and frees nothing.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two
 * streams, two threads) race and must be serialised by the caller; calls on different GPUs are independent.
 * The first call on a device looks up the array's address on that device (hipGetSymbolAddress): make one call
 * outside any capture before capturing a graph around it.
 */
int dsa_index_topk_noalloc(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu_seqlens, int T,
                           int N, int Hi, int Di, int K, float scale, int dtype, int max_seqlen, int32_t *idx,
                           int32_t *n, void *stream);
size_t dsa_index_topk_noalloc_scratch_bytes(void);
int dsa_index_topk_noalloc_max_seqlen(void);

/*
 * dsa_index_topk that also returns the indexer scores of the selected keys: sel_scores[t*K + j] = score of key
 * idx[t*K + j] (0 for j >= n[t]).  Every row is scored here, also those whose whole causal window is selected.
 * No reference counterpart (the reference holds no indexer); serves the indexer's training loss below.
 */
int dsa_index_topk_scores(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu_seqlens,
                          int T, int N, int Hi, int Di, int K, float scale, int dtype, int max_seqlen,
                          int32_t *idx, int32_t *n, float *sel_scores, void *ws, size_t ws_bytes, void *stream);

/*
 * KL divergence of the indexer's distribution over the selected keys, softmax_j(sel_scores[t,:n[t]]), from a target
 * distribution (dsa_attn_mass): loss[t] = sum_j mass (log mass - log softmax), and, when dscore != NULL, its
 * gradient w.r.t. the scores times grad_scale: (softmax - mass) * grad_scale, 0 for j >= n[t].  No reference
 * counterpart; a DSA layer adds mean(loss) to its objective in the training step (train/train_qwen.py:534-548).
 */
int dsa_indexer_kl(const float *sel_scores, const float *mass, const int32_t *n, int T, int K, float grad_scale,
                   float *loss, float *dscore, void *stream);

/*
 * Gradients of the selected indexer scores w.r.t. the indexer's inputs: given dscore[t*K + j] = dLoss/dScore of
 * key idx[t*K + j] (dsa_indexer_kl), dq_idx (T,Hi,Di) and dk_idx (T,Di) in bf16 and dw (T,Hi) in fp32, for
 * score = scale * sum_h w[t,h] relu(q_idx[t,h].k_idx[s]).  Deterministic (no atomics).  Hi <= 64, Di 64 or 128.
 * No reference counterpart (autograd of a DSA layer's indexer in the training step, train/train_qwen.py:534-548).
 */
int dsa_indexer_bwd(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *idx, const int32_t *n,
                    const float *dscore, const int32_t *cu_seqlens, int T, int N, int Hi, int Di, int K, float scale,
                    int dtype, int max_seqlen, void *dq_idx, void *dk_idx, float *dw, void *ws, size_t ws_bytes,
                    void *stream);
size_t dsa_indexer_bwd_workspace_bytes(int T, int Di, int max_seqlen);

/*
 * Stage D3 - attention forward over the selected keys (idx/n), or over every causal key of the own
 * segment when idx == NULL: that case is the drop-in for varlen_attn(..., window_size=(-1,0))
 * (train/model_attention.py:123-132; models/qwen3_vl/model.py:41-46; models/qwen3_5/model.py:93-98).
 * q head h reads kv head h / (Hq/Hkv) (models/qwen3/model.py:125-129).  softmax in fp32.
 * causal == 0 (only with idx == NULL) attends every key of the own segment: the vision towers' call,
 * varlen_attn(..., window_size=(-1,-1)) (models/qwen3_vl/model.py:423-428, models/qwen3_5/model.py:388-393).
 * head_dim D: 64, 128 or 256; with idx == NULL also 96 (forward and backward), which the 72-wide heads of the
 * 1152 / 16 vision towers are padded to.
 */
int dsa_attn_fwd(const void *q, const void *k, const void *v, const int32_t *idx, const int32_t *n,
                 const int32_t *cu_seqlens, int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale,
                 int dtype, int max_seqlen, int causal, void *out, float *lse, void *ws, size_t ws_bytes, void *stream);

/*
 * The selection bitmap without a pass over the finished list (no reference counterpart).  dsa_index_topk_bitmap is
 * dsa_index_topk (sel_scores == NULL) or dsa_index_topk_scores (sel_scores != NULL) whose top-k kernel also leaves,
 * in `bitmap`, what dsa_attn_fwd would build from idx/n in its workspace (same layout and size:
 * dsa_attn_fwd_workspace_bytes(T, max_seqlen, 1)) - the ballots of its compaction are those words already.
 * dsa_attn_fwd_saved_bitmap is dsa_attn_fwd reading such a bitmap (made with the same idx, n, cu_seqlens and
 * max_seqlen by dsa_index_topk_bitmap or by an earlier dsa_attn_fwd) instead of building it; the same buffer then
 * serves dsa_attn_bwd_saved_bitmap.  With the tile crossover at 0 no kernel reads the bitmap.
 */
int dsa_index_topk_bitmap(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu_seqlens, int T, int N,
                          int Hi, int Di, int K, float scale, int dtype, int max_seqlen, int32_t *idx, int32_t *n,
                          float *sel_scores, void *bitmap, size_t bitmap_bytes, void *ws, size_t ws_bytes, void *stream);
int dsa_attn_fwd_saved_bitmap(const void *q, const void *k, const void *v, const int32_t *idx, const int32_t *n,
                              const int32_t *cu_seqlens, int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale,
                              int dtype, int max_seqlen, int causal, void *out, float *lse, const void *bitmap,
                              size_t bitmap_bytes, void *stream);

/* Bytes of workspace dsa_attn_fwd needs (the inverted selection bitmap; 0 without idx). */
size_t dsa_attn_fwd_workspace_bytes(int T, int max_seqlen, int has_idx);

/*
 * Attention mass of the selected keys: mass[t*K + j] = 1/Hq * sum over query heads of the softmax
 * probability that D3 gave key idx[t*K + j] (lse is D3's output), 0 for j >= n[t].  Every head's softmax
 * over sel(t) sums to one, so a row sums to one: it is the target distribution of the KL loss that
 * trains a DSA indexer (the selection itself passes no gradient).  No reference counterpart - the
 * reference holds no indexer; it would be called beside the attention call of a layer in its training
 * step (train/train_qwen.py:534-548).  fp32 out, deterministic.  ws: dsa_attn_mass_workspace_bytes() for the
 * same geometry: the selection bitmap and one (T,K) fp32 table per group of kv heads - a workgroup takes the kv
 * heads of its group in turn and sums in place; one to Hkv groups, as many as fill the chip (two at 32 768 tokens
 * with 8 kv heads: 0.5 GiB; none when one group takes every kv head).
 */
int dsa_attn_mass(const void *q, const void *k, const float *lse, const int32_t *idx, const int32_t *n,
                  const int32_t *cu_seqlens, int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale,
                  int dtype, int max_seqlen, float *mass, void *ws, size_t ws_bytes, void *stream);
size_t dsa_attn_mass_workspace_bytes(int T, int N, int Hq, int Hkv, int D, int K, int max_seqlen);
/* dsa_attn_mass reading the selection bitmap that dsa_index_topk_bitmap or a forward left (the same idx, n, cu_seqlens
 * and max_seqlen) instead of building its own; ws then holds only what dsa_attn_mass_workspace_bytes() asks for beyond
 * dsa_attn_fwd_workspace_bytes(T, max_seqlen, 1) - nothing at all where one workgroup holds every kv head (ws may be
 * NULL then). */
int dsa_attn_mass_saved_bitmap(const void *q, const void *k, const float *lse, const int32_t *idx, const int32_t *n,
                               const int32_t *cu_seqlens, int T, int N, int Hq, int Hkv, int D, int K,
                               float softmax_scale, int dtype, int max_seqlen, float *mass, const void *bitmap,
                               size_t bitmap_bytes, void *ws, size_t ws_bytes, void *stream);

/*
 * Tuning knob (process-wide, no reference counterpart): query rows whose position in their segment is
 * below top_k * crossover run on the dense MFMA tile kernels with the selection as a bitmap mask, the
 * rest on the gather kernels.  Default 24 (one 131 072-token sequence with top-k 2048: forward 115 -> 110 ms and
 * dQ 123 -> 120 ms against 16; 32 is level with it); 0 = gather only; INT_MAX/top_k or more = tiles only.
 * idx == NULL (dense causal attention) always uses the tile kernels.
 */
int dsa_set_tile_crossover(int crossover);
int dsa_get_tile_crossover(void);

/*
 * Tuning knob (process-wide, no reference counterpart): the backward's query-side pass (dQ) and key-side pass (dK/dV)
 * read the same inputs and write different outputs.  1 (default): when the key-side launch has at most 1536
 * workgroups - a short batch, or one GPU's share of head-sharded attention, which ends on its longest walks with most
 * CUs idle - and T * max_seqlen * Hq * D is at least 6e10 (below that the fork and join cost what the overlap gains)
 * the query side runs on a second stream of the library's own (default priority, one per device, created
 * on the first such call outside a capture) between a fork and a join event on the caller's stream, so that to the
 * caller the whole call is still ordered on the stream it passed; under stream capture the second stream joins the
 * capture through those events.  0: never (one stream).  2: for every launch size.  Results are the same bits in all
 * modes.  dsa_indexer_bwd runs its query side and its key side the same way (mode 1: up to 16 384 tokens).
 */
int dsa_set_bwd_overlap(int mode);
int dsa_get_bwd_overlap(void);

/* Bytes of workspace dsa_attn_bwd needs: softmax row terms, the inverted selection bitmap, the launch order of the
 * dK/dV key tiles (about 128 KiB + T/8 bytes) and, up to 131072 tokens, fp32 partial sums for key-tile walks that a
 * small launch cuts into pieces (16 KiB per token, at most 128 MiB). */
size_t dsa_attn_bwd_workspace_bytes(int T, int Hq, int max_seqlen, int has_idx);
/*
 * Byte offset of the selection bitmap inside the backward workspace.  A forward call handed
 * `ws + offset` as its workspace leaves the bitmap where a later dsa_attn_bwd_parts on the same `ws`
 * finds it, so that backward can be run without DSA_BWD_BITMAP (the autograd wrapper does this).
 * No reference counterpart: the reference's attention saves no selection.
 */
size_t dsa_attn_bwd_bitmap_offset(int T, int Hq);

/*
 * Stage D4 - gradients of D3 (the autograd backward of varlen_attn restricted to the selected keys;
 * aten::_flash_attention_backward in the reference's stack).  Deterministic: no atomics on dq/dk/dv.
 */
int dsa_attn_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out, const float *lse,
                 const int32_t *idx, const int32_t *n, const int32_t *cu_seqlens, int T, int N, int Hq, int Hkv,
                 int D, int K, float softmax_scale, int dtype, int max_seqlen, int causal, void *dq, void *dk,
                 void *dv, void *ws, size_t ws_bytes, void *stream);

/*
 * Measurement hook: dsa_attn_bwd restricted to the kernels named in `parts`, so that each can be
 * timed on its own with events on the caller's stream.  Parts must be run in bit order at least once
 * on the same workspace before a later part is timed alone (the later kernels read what the earlier
 * ones leave in ws).  No reference counterpart.
 */
#define DSA_BWD_DELTA 1  /* delta = rowsum(dO * O) */
#define DSA_BWD_BITMAP 2 /* inverted selection bitmap (only when idx != NULL) */
#define DSA_BWD_DQ 4     /* query-side pass (tile and/or gather kernel) */
#define DSA_BWD_DKV 8    /* key-side pass */
#define DSA_BWD_ALL 15
int dsa_attn_bwd_parts(const void *dout, const void *q, const void *k, const void *v, const void *out,
                       const float *lse, const int32_t *idx, const int32_t *n, const int32_t *cu_seqlens, int T, int N,
                       int Hq, int Hkv, int D, int K, float softmax_scale, int dtype, int max_seqlen, int causal,
                       void *dq, void *dk, void *dv, void *ws, size_t ws_bytes, int parts, void *stream);

/*
 * dsa_attn_bwd for a caller that kept the forward's workspace (an autograd node: torch's varlen_attn saves its
 * tensors between forward and backward the same way, torch/nn/attention/varlen.py:206-214).  `fwd_ws` is the
 * workspace a dsa_attn_fwd call with the same idx, n, cu_seqlens and max_seqlen filled (the inverted selection
 * bitmap; ignored when idx == NULL); it is only read.  `scratch` holds dsa_attn_bwd_scratch_bytes() bytes that
 * nothing outlives: delta, the launch order of the key tiles and - only for launches of at most 1024 key-tile
 * workgroups, which may be cut into pieces - fp32 partial sums (at most 128 MiB).  So between forward and backward
 * a layer holds the bitmap alone.  Refused (DSA_ERR_ARG) while the tile crossover is 0: that forward builds no bitmap.
 */
size_t dsa_attn_bwd_scratch_bytes(int T, int N, int Hq, int Hkv, int D);
int dsa_attn_bwd_saved_bitmap(const void *dout, const void *q, const void *k, const void *v, const void *out,
                              const float *lse, const int32_t *idx, const int32_t *n, const int32_t *cu_seqlens, int T,
                              int N, int Hq, int Hkv, int D, int K, float softmax_scale, int dtype, int max_seqlen,
                              int causal, void *dq, void *dk, void *dv, const void *fwd_ws, size_t fwd_ws_bytes,
                              void *scratch, size_t scratch_bytes, void *stream);

/*
 * Dense causal / non-causal packed attention, the operator the reference itself calls
 * (torch.nn.attention.varlen.varlen_attn: train/model_attention.py:123-132, models/qwen3_vl/model.py:41-46,
 * models/qwen3_5/model.py:93-98).  Same as dsa_attn_fwd / dsa_attn_bwd with idx == n == NULL and K == 0;
 * no workspace is needed forward, dsa_attn_bwd_workspace_bytes(T, Hq, max_seqlen, 0) bytes backward.
 */
int dsa_dense_fwd(const void *q, const void *k, const void *v, const int32_t *cu_seqlens, int T, int N, int Hq, int Hkv,
                  int D, float softmax_scale, int dtype, int max_seqlen, int causal, void *out, float *lse, void *stream);
int dsa_dense_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out, const float *lse,
                  const int32_t *cu_seqlens, int T, int N, int Hq, int Hkv, int D, float softmax_scale, int dtype,
                  int max_seqlen, int causal, void *dq, void *dk, void *dv, void *ws, size_t ws_bytes, void *stream);

/* ---------------------------------------------------------------------------------------------------
 * Pre-attention prologue and post-attention gate (the element-wise work either side of the operator).
 *
 * dsa_qk_norm_rope_fwd stands for, in one pass over q and k (models/qwen3_vl/model.py:256-269,
 * models/qwen3_5/model.py:110-129): `q_norm(q)`, `k_norm(k)` = F.rms_norm over head_dim with weight `w`
 * or `1 + w` (`norm_flags & DSA_NORM_OFFSET`: OffsetRMSNorm, models/qwen3_5/model.py:58-72), the two
 * transposes, `apply_rope(q, k, cos, sin)` (models/qwen3_vl/model.py:181-193; partial rotary width
 * R <= D: models/qwen3_5/utils.py:88-110) and the `.contiguous()` copies into (T, H, D).
 *   q_in, k_in: bf16, element (t, h, d) at  base + t*tok_stride + h*head_stride + d  (strides in elements,
 *               so the q half of Qwen3.5's interleaved [q | gate] projection can be read in place);
 *   qw, kw: (D) fp32, or bf16 with `norm_flags & DSA_NORM_WEIGHT_BF16` (read as the module holds them: no cast
 *           kernel in front of the call);  cos, sin: (T, R) bf16 (cs_dtype DSA_DTYPE_BF16) or fp32 (DSA_DTYPE_FP32), R % 16 == 0;
 *   q_out (T,Hq,D), k_out (T,Hkv,D) bf16 contiguous;  q_rstd (T,Hq), k_rstd (T,Hkv) fp32: 1/rms of
 *   every row, kept for the backward pass.  D in {64, 128, 256}.
 * dsa_qk_norm_rope_bwd: gq, gk = gradients of q_out, k_out (same layout) -> dq_in, dk_in (strided like
 * the inputs, bf16) and dqw, dkw (D) fp32.  `ws` holds dsa_qk_norm_rope_bwd_workspace_bytes(T, D) bytes
 * of per-workgroup partial sums that are added up in a fixed order (no atomics, deterministic).
 */
#define DSA_NORM_OFFSET 1      /* scale by 1 + w */
#define DSA_NORM_WEIGHT_BF16 2 /* qw, kw point at bf16 */
size_t dsa_qk_norm_rope_bwd_workspace_bytes(int T, int D);
int dsa_qk_norm_rope_fwd(const void *q_in, int64_t q_tok_stride, int64_t q_head_stride, const void *k_in,
                         int64_t k_tok_stride, int64_t k_head_stride, const void *qw, const void *kw, float eps,
                         int norm_flags, const void *cos, const void *sin, int cs_dtype, int R, int T, int Hq, int Hkv,
                         int D, void *q_out, void *k_out, float *q_rstd, float *k_rstd, void *stream);
int dsa_qk_norm_rope_bwd(const void *gq, const void *gk, const void *q_in, int64_t q_tok_stride, int64_t q_head_stride,
                         const void *k_in, int64_t k_tok_stride, int64_t k_head_stride, const void *qw, const void *kw,
                         int norm_flags, const void *cos, const void *sin, int cs_dtype, int R, const float *q_rstd,
                         const float *k_rstd, int T, int Hq, int Hkv, int D, void *dq_in, int64_t dq_tok_stride,
                         int64_t dq_head_stride, void *dk_in, int64_t dk_tok_stride, int64_t dk_head_stride, float *dqw,
                         float *dkw, void *ws, size_t ws_bytes, void *stream);
/*
 * `out * torch.sigmoid(gate)` (models/qwen3_5/model.py:135) and its gradients.  x, y, gy, dx: (T, H, D)
 * bf16 contiguous; gate and dgate: element (t, h, d) at base + t*tok_stride + h*head_stride + d.
 */
int dsa_sigmoid_gate_fwd(const void *x, const void *gate, int64_t gate_tok_stride, int64_t gate_head_stride, int T,
                         int H, int D, void *y, void *stream);
int dsa_sigmoid_gate_bwd(const void *gy, const void *x, const void *gate, int64_t gate_tok_stride,
                         int64_t gate_head_stride, int T, int H, int D, void *dx, void *dgate, int64_t dgate_tok_stride,
                         int64_t dgate_head_stride, void *stream);

/*
 * fp32 operands on the bf16 kernels (no reference counterpart: the reference runs the operator in bf16 under autocast;
 * this serves fp32 callers such as the CPU-runnable toy configuration).  x (rows, D) fp32 -> y (rows, 4*D) bf16 holding
 * hi = bf16(x) and lo = bf16(x - hi) stacked along the last dimension: order 0 = [hi, lo, hi, 0] (q, v), order 1 =
 * [hi, hi, lo, 0] (k, dO), so that <q', k'> = <q, k> - <q_lo, k_lo>.  dsa_split_bf16_combine is the way back:
 * out[r, :] = y[r, 0:D] + y[r, part*D:(part+1)*D] in fp32 (part 1: out, dk; part 2: dq, dv).  D % 4 == 0.
 */
int dsa_split_bf16_stack(const float *x, int64_t rows, int D, int order, void *y, void *stream);
int dsa_split_bf16_combine(const void *y, int64_t rows, int D, int part, float *out, void *stream);
/* The three operands of one attention call in one launch: q (rows_q, D) with order 0, k (rows_kv, D) with order 1 and
 * v (rows_kv, D) with order 0; and the way back for the three gradients: dq part 2, dk part 1, dv part 2. */
int dsa_split_bf16_stack_qkv(const float *q, const float *k, const float *v, int64_t rows_q, int64_t rows_kv, int D,
                             void *yq, void *yk, void *yv, void *stream);
int dsa_split_bf16_combine_qkv(const void *yq, const void *yk, const void *yv, int64_t rows_q, int64_t rows_kv, int D,
                               float *dq, float *dk, float *dv, void *stream);

/*
 * Three fp32 arrays of na, nb, nc elements rounded to bf16 (to nearest even, what tensor.to(torch.bfloat16) gives) by one
 * launch: the indexer's three inputs when the caller holds them in fp32 (no reference counterpart: the reference runs
 * under bf16 autocast).  Inputs 16-byte aligned, outputs 8-byte aligned.
 */
int dsa_round_bf16_x3(const float *a, const float *b, const float *c, int64_t na, int64_t nb, int64_t nc, void *ya, void *yb,
                      void *yc, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DSA_ATTN_H */
