// C ABI of the library (declared in include/dsa_attn.h): argument checks, workspace layout, launches.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <mutex>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../../include/dsa_attn.h"

extern "C" {
hipError_t dsa_launch_topk(const float *scores, int64_t ld, int row_begin, int row_end, const int32_t *cu, int N,
                           int K, int max_row, int32_t *idx, int32_t *n, uint32_t *bitmap, int ldw, float *sel, hipStream_t stream);
hipError_t dsa_launch_indexer_kl(const float *sel, const float *mass, const int32_t *n, int T, int K, float grad_scale,
                                 float *loss, float *dscore, hipStream_t stream);
hipError_t dsa_launch_indexer(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu, int N,
                              int T, int Hi, int Di, float scale, int row_begin, int row_end, int skip_dense_k,
                              float *scores, int64_t ld, hipStream_t stream);
hipError_t dsa_launch_attn_fwd(const void *q, const void *k, const void *v, const int32_t *idx, const int32_t *n,
                               const int32_t *cu, int N, int T, int Hq, int Hkv, int D, int K, float scale, int pos_min,
                               void *out, float *lse, hipStream_t stream);
hipError_t dsa_launch_delta(const void *dout, const void *out, int T, int Hq, int D, float *delta, hipStream_t stream);
hipError_t dsa_launch_bitmap(const int32_t *idx, const int32_t *n, const int32_t *cu, int N, int T, int K, int ldw,
                             uint32_t *bitmap, hipStream_t stream);
hipError_t dsa_launch_gather_dq(const void *dout, const void *q, const void *k, const void *v, const float *lse,
                                const float *delta, const int32_t *idx, const int32_t *n, const int32_t *cu, int N,
                                int T, int Hq, int Hkv, int D, int K, float scale, int pos_min, void *dq,
                                hipStream_t stream);
hipError_t dsa_launch_indexer_bwd(const void *q_idx, const void *k_idx, const void *w_idx, const float *dscore,
                                  const uint32_t *bitmap, int32_t *prefix, int ldw, const int32_t *cu, int N, int T, int Hi,
                                  int Di, int K, float cscale, void *dq_idx, void *dk_idx, float *dw, float *partial,
                                  hipStream_t stream, hipStream_t stream_q);
size_t dsa_indexer_bwd_partial_bytes(int T, int Di, int ldw);
hipError_t dsa_launch_tile_mass(const void *q, const void *k, const float *lse, const uint32_t *bitmap, int ldw,
                                const int32_t *n, const int32_t *cu, int N, int T, int Hq, int Hkv, int D, int K,
                                float scale, float *partial, float *mass, hipStream_t stream);
hipError_t dsa_launch_tile_fwd(const void *q, const void *k, const void *v, const uint32_t *bitmap, int ldw,
                               const int32_t *cu, int N, int T, int Hq, int Hkv, int D, float scale, int pos_split,
                               int causal, void *out, float *lse, hipStream_t stream);
hipError_t dsa_launch_tile_dq(const void *dout, const void *q, const void *k, const void *v, const float *lse,
                              const float *delta, const uint32_t *bitmap, int ldw, const int32_t *cu, int N, int T,
                              int Hq, int Hkv, int D, float scale, int pos_split, int causal, void *dq, const void *out_for_delta,
                              float *delta_out, hipStream_t stream);
hipError_t dsa_launch_tile_dkv(const void *dout, const void *q, const void *k, const void *v, const float *lse,
                               const float *delta, const uint32_t *bitmap, int ldw, const int32_t *cu, int N, int T,
                               int Hq, int Hkv, int D, float scale, int causal, int32_t *order, float *partial,
                               size_t partial_bytes, void *dk, void *dv, hipStream_t stream);
size_t dsa_tile_order_bytes(int T);
size_t dsa_tile_dkv_partial_bytes(int T);
int dsa_mass_groups(int Hq, int Hkv, int D);
}

extern "C" {
int dsa_prologue_bwd_blocks(int T);
hipError_t dsa_launch_qk_norm_rope_fwd(const void *q_in, int64_t q_tok, int64_t q_head, const void *k_in, int64_t k_tok,
                                       int64_t k_head, const void *qw, const void *kw, int w_bf16, float eps, float w_offset,
                                       const void *cosp, const void *sinp, int cs_f32, int R, int T, int Hq, int Hkv, int D,
                                       void *q_out, void *k_out, float *q_rstd, float *k_rstd, hipStream_t stream);
hipError_t dsa_launch_qk_norm_rope_bwd(const void *gq, const void *gk, const void *q_in, int64_t q_tok, int64_t q_head,
                                       const void *k_in, int64_t k_tok, int64_t k_head, const void *qw, const void *kw,
                                       int w_bf16, float w_offset, const void *cosp, const void *sinp, int cs_f32, int R,
                                       const float *q_rstd, const float *k_rstd, int T, int Hq, int Hkv, int D, void *dq_in,
                                       int64_t dq_tok, int64_t dq_head, void *dk_in, int64_t dk_tok, int64_t dk_head,
                                       float *dqw, float *dkw, float *part, hipStream_t stream);
hipError_t dsa_launch_sigmoid_gate_fwd(const void *x, const void *gate, int64_t gate_tok, int64_t gate_head, int D, int H,
                                       int64_t rows, void *y, hipStream_t stream);
hipError_t dsa_launch_split_stack(const float *x, int64_t rows, int D, int order, void *y, hipStream_t stream);
hipError_t dsa_launch_split_combine(const void *y, int64_t rows, int D, int part, float *out, hipStream_t stream);
hipError_t dsa_launch_round_bf16_x3(const float *a, const float *b, const float *c, int64_t na, int64_t nb, int64_t nc, void *ya,
                                    void *yb, void *yc, hipStream_t stream);
hipError_t dsa_launch_split_stack_qkv(const float *q, const float *k, const float *v, int64_t rows_q, int64_t rows_kv, int D, void *yq,
                                      void *yk, void *yv, hipStream_t stream);
hipError_t dsa_launch_split_combine_qkv(const void *yq, const void *yk, const void *yv, int64_t rows_q, int64_t rows_kv, int D,
                                        float *dq, float *dk, float *dv, hipStream_t stream);
hipError_t dsa_launch_sigmoid_gate_bwd(const void *gy, const void *x, const void *gate, int64_t gate_tok, int64_t gate_head,
                                       int D, int H, int64_t rows, void *dx, void *dgate, int64_t dgate_tok,
                                       int64_t dgate_head, hipStream_t stream);
}

static thread_local char g_err[512] = "";

static int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}
static int hip_fail(hipError_t e, const char *what) {
    return fail(DSA_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}
static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

#define SCORE_CHUNK_BYTES ((size_t)1 << 30)
static inline int64_t score_ld(int max_seqlen) { return (int64_t)align_up((size_t)max_seqlen, 32); }

extern "C" const char *dsa_version(void) { return "dsa-attn-gfx950 0.1"; }
extern "C" const char *dsa_last_error(void) { return g_err; }

static int check_packed(int T, int N, const int32_t *cu) {
    if (T < 0 || N < 1) return fail(DSA_ERR_ARG, "T=%d N=%d: need T>=0 and at least one segment", T, N);
    if (!cu) return fail(DSA_ERR_ARG, "cu_seqlens is null");
    return DSA_OK;
}

extern "C" int dsa_indexer_scores(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu, int T,
                                  int N, int Hi, int Di, float scale, int dtype, int row_begin, int row_end,
                                  int skip_dense_k, float *scores, int64_t ld, void *stream) {
    if (int rc = check_packed(T, N, cu)) return rc;
    if (dtype != DSA_DTYPE_BF16) return fail(DSA_ERR_UNSUPPORTED, "indexer inputs must be bf16 (dtype code %d)", dtype);
    if (!q_idx || !k_idx || !w_idx || !scores) return fail(DSA_ERR_ARG, "null tensor pointer");
    if (row_begin < 0 || row_end > T || row_begin > row_end) return fail(DSA_ERR_ARG, "bad row range [%d,%d)", row_begin, row_end);
    if (Hi < 1 || Hi > 64 || !(Di == 32 || Di == 64 || Di == 128))
        return fail(DSA_ERR_UNSUPPORTED, "indexer geometry Hi=%d Di=%d: need Hi<=64 and Di in {32,64,128}", Hi, Di);
    hipError_t e = dsa_launch_indexer(q_idx, k_idx, w_idx, cu, N, T, Hi, Di, scale, row_begin, row_end, skip_dense_k,
                                      scores, ld, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "indexer launch");
}

extern "C" int dsa_topk_from_scores(const float *scores, int64_t ld, int row_begin, int row_end, const int32_t *cu,
                                    int T, int N, int K, int32_t *idx, int32_t *n, void *stream) {
    if (int rc = check_packed(T, N, cu)) return rc;
    if (!scores || !idx || !n) return fail(DSA_ERR_ARG, "null tensor pointer");
    if (K < 1) return fail(DSA_ERR_ARG, "top_k=%d must be >= 1", K);
    if (row_begin < 0 || row_end > T || row_begin > row_end) return fail(DSA_ERR_ARG, "bad row range [%d,%d)", row_begin, row_end);
    hipError_t e = dsa_launch_topk(scores, ld, row_begin, row_end, cu, N, K, (int)ld, idx, n, nullptr, 0, nullptr, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "top-k launch");
}

extern "C" size_t dsa_index_topk_workspace_bytes(int T, int max_seqlen, int K) {
    (void)K;
    if (T <= 0 || max_seqlen <= 0) return 0;
    const size_t row_bytes = (size_t)score_ld(max_seqlen) * 4;
    size_t rows = SCORE_CHUNK_BYTES / row_bytes;
    if (rows < 64) rows = 64;
    if (rows > (size_t)T) rows = (size_t)T;
    return align_up(rows, 4) * row_bytes;
}

static inline int bitmap_ldw(int max_seqlen) { return (max_seqlen + 31) / 32; }   // words of a row of the selection bitmap

// sel_scores != NULL: every row is scored (also those whose whole causal window is selected) and the scores of
// the selected keys are kept; bitmap != NULL: the top-k kernel also leaves the inverted selection there
static int index_topk_impl(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu, int T, int N,
                           int Hi, int Di, int K, float scale, int dtype, int max_seqlen, int32_t *idx, int32_t *n,
                           float *sel_scores, uint32_t *bitmap, void *ws, size_t ws_bytes, void *stream) {
    if (int rc = check_packed(T, N, cu)) return rc;
    if (K < 1) return fail(DSA_ERR_ARG, "top_k=%d must be >= 1", K);
    if (max_seqlen < 1 || max_seqlen > T) return fail(DSA_ERR_ARG, "max_seqlen=%d outside [1,T=%d]", max_seqlen, T);
    if (!idx || !n) return fail(DSA_ERR_ARG, "null output pointer");
    if (T == 0) return DSA_OK;
    const int64_t ld = score_ld(max_seqlen);
    int64_t rows = ws ? (int64_t)(ws_bytes / ((size_t)ld * 4)) : 0;
    rows &= ~(int64_t)3;
    if (max_seqlen <= K && !sel_scores) rows = T;   // every row is dense: no score is read or written
    else if (rows < 4) return fail(DSA_ERR_WORKSPACE, "workspace of %zu bytes holds no score chunk (row = %lld bytes)", ws_bytes, (long long)ld * 4);
    if (rows > T) rows = T;
    for (int64_t r0 = 0; r0 < T; r0 += rows) {
        const int r1 = (int)((r0 + rows < T) ? r0 + rows : T);
        if (max_seqlen > K || sel_scores) {
            int rc = dsa_indexer_scores(q_idx, k_idx, w_idx, cu, T, N, Hi, Di, scale, dtype, (int)r0, r1, sel_scores ? 0 : K,
                                        (float *)ws, ld, stream);
            if (rc) return rc;
        }
        hipError_t e = dsa_launch_topk((const float *)ws, ld, (int)r0, r1, cu, N, K, max_seqlen, idx, n, bitmap,
                                       bitmap_ldw(max_seqlen), sel_scores, (hipStream_t)stream);
        if (e != hipSuccess) return hip_fail(e, "top-k launch");
    }
    return DSA_OK;
}

extern "C" int dsa_index_topk(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu, int T, int N,
                              int Hi, int Di, int K, float scale, int dtype, int max_seqlen, int32_t *idx, int32_t *n,
                              void *ws, size_t ws_bytes, void *stream) {
    return index_topk_impl(q_idx, k_idx, w_idx, cu, T, N, Hi, Di, K, scale, dtype, max_seqlen, idx, n, nullptr, nullptr, ws,
                           ws_bytes, stream);
}

extern "C" int dsa_index_topk_scores(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu, int T,
                                     int N, int Hi, int Di, int K, float scale, int dtype, int max_seqlen, int32_t *idx,
                                     int32_t *n, float *sel_scores, void *ws, size_t ws_bytes, void *stream) {
    if (!sel_scores) return fail(DSA_ERR_ARG, "null output pointer");
    return index_topk_impl(q_idx, k_idx, w_idx, cu, T, N, Hi, Di, K, scale, dtype, max_seqlen, idx, n, sel_scores, nullptr,
                           ws, ws_bytes, stream);
}

// ---- dsa_index_topk for callers that cannot allocate -------------------------------------------------------
// The score rows live in a file-scope device array instead of a caller's workspace.  Its name is a host-side handle,
// not a device address: the address is looked up once per device (every GPU holds its own copy of the array) and only
// that pointer is ever handed to a kernel.
#define DSA_SCRATCH_BYTES ((size_t)32 << 20)
#define DSA_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[DSA_SCRATCH_BYTES];
static void *g_scratch_ptr[DSA_MAX_DEVICES];
static std::mutex g_scratch_mu;

static int scratch_of_current_device(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= DSA_MAX_DEVICES) return fail(DSA_ERR_UNSUPPORTED, "device %d: the static scratch serves devices 0..%d", dev, DSA_MAX_DEVICES - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return DSA_OK;
}

extern "C" size_t dsa_index_topk_noalloc_scratch_bytes(void) { return DSA_SCRATCH_BYTES; }
// longest segment whose four score rows (the smallest chunk the chunked loop works on) fit the scratch
extern "C" int dsa_index_topk_noalloc_max_seqlen(void) { return (int)(DSA_SCRATCH_BYTES / (4 * sizeof(float)) / 32 * 32); }

extern "C" int dsa_index_topk_noalloc(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu, int T,
                                      int N, int Hi, int Di, int K, float scale, int dtype, int max_seqlen, int32_t *idx,
                                      int32_t *n, void *stream) {
    if (max_seqlen > dsa_index_topk_noalloc_max_seqlen())
        return fail(DSA_ERR_WORKSPACE, "max_seqlen=%d: the %zu-byte static scratch holds score rows of at most %d columns; "
                    "use dsa_index_topk with a workspace of your own", max_seqlen, DSA_SCRATCH_BYTES,
                    dsa_index_topk_noalloc_max_seqlen());
    void *ws = nullptr;
    if (int rc = scratch_of_current_device(&ws)) return rc;
    // nothing in the scratch has to start at zero: the indexer writes every column [0, pos] of a row before the
    // selection reads it, and rows whose whole window is selected are never read
    return index_topk_impl(q_idx, k_idx, w_idx, cu, T, N, Hi, Di, K, scale, dtype, max_seqlen, idx, n, nullptr, nullptr, ws,
                           DSA_SCRATCH_BYTES, stream);
}

extern "C" int dsa_indexer_kl(const float *sel_scores, const float *mass, const int32_t *n, int T, int K, float grad_scale,
                              float *loss, float *dscore, void *stream) {
    if (T < 0 || K < 1) return fail(DSA_ERR_ARG, "T=%d, top_k=%d", T, K);
    if (T > 0 && (!sel_scores || !mass || !n || !loss)) return fail(DSA_ERR_ARG, "null tensor pointer");
    hipError_t e = dsa_launch_indexer_kl(sel_scores, mass, n, T, K, grad_scale, loss, dscore, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "indexer KL launch");
}

static int check_attn(int T, int N, const int32_t *cu, int Hq, int Hkv, int D, int K, int dtype, const int32_t *idx,
                      const int32_t *n) {
    if (int rc = check_packed(T, N, cu)) return rc;
    if (dtype != DSA_DTYPE_BF16) return fail(DSA_ERR_UNSUPPORTED, "q/k/v must be bf16 (dtype code %d)", dtype);
    if (Hq < 1 || Hkv < 1 || Hq % Hkv) return fail(DSA_ERR_ARG, "Hq=%d must be a positive multiple of Hkv=%d", Hq, Hkv);
    if (Hq / Hkv > 16) return fail(DSA_ERR_UNSUPPORTED, "Hq/Hkv=%d: at most 16 query heads per kv head", Hq / Hkv);
    if (!(D == 64 || D == 128 || D == 256 || (D == 96 && !idx)))
        return fail(DSA_ERR_UNSUPPORTED, "head_dim=%d: need 64, 128 or 256 (96 as well without a key selection)", D);
    if ((idx == nullptr) != (n == nullptr)) return fail(DSA_ERR_ARG, "idx and n must both be given or both be null");
    if (idx && K < 1) return fail(DSA_ERR_ARG, "top_k=%d must be >= 1", K);
    if ((int64_t)T * Hkv >= ((int64_t)1 << 31)) return fail(DSA_ERR_UNSUPPORTED, "T*Hkv too large for one launch");
    return DSA_OK;
}

// Query rows whose position in their segment is below top_k * crossover are handled by the tile
// kernels (their selection covers more than 1/crossover of the causal window), the rest by the
// gather kernels.  Process-wide tuning knob; 0 = gather only, a huge value = tile only.
static std::atomic<int> g_tile_crossover{24};          // read on every launch, possibly from several host threads
extern "C" int dsa_set_tile_crossover(int crossover) {
    if (crossover < 0) return fail(DSA_ERR_ARG, "crossover=%d must be >= 0", crossover);
    g_tile_crossover.store(crossover, std::memory_order_relaxed);
    return DSA_OK;
}
extern "C" int dsa_get_tile_crossover(void) { return g_tile_crossover.load(std::memory_order_relaxed); }

// first query position handled by the gather kernels (multiple of 128, the coarsest tile block)
static int pos_split_for(const int32_t *idx, int K) {
    if (!idx) return INT32_MAX;                       // dense causal: tiles everywhere
    const int64_t p = (int64_t)K * g_tile_crossover.load(std::memory_order_relaxed);
    if (p >= INT32_MAX - 256) return INT32_MAX;
    return (int)((p + 255) / 256 * 256);          // a multiple of every tile kernel's query block
}

extern "C" size_t dsa_attn_fwd_workspace_bytes(int T, int max_seqlen, int has_idx) {
    if (T <= 0 || !has_idx) return 0;
    return align_up((size_t)T * bitmap_ldw(max_seqlen) * 4, 256);
}

// build_bitmap == 0: ws already holds the bitmap of idx/n (it is only read)
static int attn_fwd_run(const void *q, const void *k, const void *v, const int32_t *idx, const int32_t *n, const int32_t *cu,
                        int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale, int dtype, int max_seqlen, int causal,
                        void *out, float *lse, void *ws, size_t ws_bytes, int build_bitmap, void *stream) {
    if (int rc = check_attn(T, N, cu, Hq, Hkv, D, K, dtype, idx, n)) return rc;
    if (!causal && idx) return fail(DSA_ERR_ARG, "a key selection (idx) implies causal attention");
    if (!q || !k || !v || !out || !lse) return fail(DSA_ERR_ARG, "null tensor pointer");
    if (max_seqlen < 1 || max_seqlen > (T > 0 ? T : 1)) return fail(DSA_ERR_ARG, "max_seqlen=%d outside [1,T=%d]", max_seqlen, T);
    if (T == 0) return DSA_OK;
    const int split = pos_split_for(idx, K);
    const int ldw = bitmap_ldw(max_seqlen);
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = hipSuccess;
    if (split > 0) {
        uint32_t *bitmap = nullptr;
        if (idx) {
            const size_t need = dsa_attn_fwd_workspace_bytes(T, max_seqlen, 1);
            if (!ws || ws_bytes < need) return fail(DSA_ERR_WORKSPACE, "forward workspace: have %zu bytes, need %zu", ws_bytes, need);
            if ((size_t)ldw * 4 > 64 * 1024) return fail(DSA_ERR_UNSUPPORTED, "max_seqlen=%d: selection bitmap row exceeds 64 KiB of LDS", max_seqlen);
            bitmap = (uint32_t *)ws;
            if (build_bitmap) {
                e = dsa_launch_bitmap(idx, n, cu, N, T, K, ldw, bitmap, st);
                if (e != hipSuccess) return hip_fail(e, "bitmap launch");
            }
        }
        e = dsa_launch_tile_fwd(q, k, v, bitmap, ldw, cu, N, T, Hq, Hkv, D, softmax_scale, split, causal, out, lse, st);
        if (e != hipSuccess) return hip_fail(e, "tile forward launch");
    }
    if (max_seqlen > split) {
        e = dsa_launch_attn_fwd(q, k, v, idx, n, cu, N, T, Hq, Hkv, D, K, softmax_scale, split, out, lse, st);
        if (e != hipSuccess) return hip_fail(e, "gather forward launch");
    }
    return DSA_OK;
}

extern "C" int dsa_attn_fwd(const void *q, const void *k, const void *v, const int32_t *idx, const int32_t *n,
                            const int32_t *cu, int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale,
                            int dtype, int max_seqlen, int causal, void *out, float *lse, void *ws, size_t ws_bytes,
                            void *stream) {
    return attn_fwd_run(q, k, v, idx, n, cu, T, N, Hq, Hkv, D, K, softmax_scale, dtype, max_seqlen, causal, out, lse, ws, ws_bytes,
                        1, stream);
}

extern "C" int dsa_attn_fwd_saved_bitmap(const void *q, const void *k, const void *v, const int32_t *idx, const int32_t *n,
                                         const int32_t *cu, int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale,
                                         int dtype, int max_seqlen, int causal, void *out, float *lse, const void *bitmap,
                                         size_t bitmap_bytes, void *stream) {
    if (!idx) return fail(DSA_ERR_ARG, "a saved bitmap belongs to a selection: idx is null");
    return attn_fwd_run(q, k, v, idx, n, cu, T, N, Hq, Hkv, D, K, softmax_scale, dtype, max_seqlen, causal, out, lse,
                        const_cast<void *>(bitmap), bitmap_bytes, 0, stream);
}

extern "C" int dsa_index_topk_bitmap(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu, int T, int N,
                                     int Hi, int Di, int K, float scale, int dtype, int max_seqlen, int32_t *idx, int32_t *n,
                                     float *sel_scores, void *bitmap, size_t bitmap_bytes, void *ws, size_t ws_bytes,
                                     void *stream) {
    if (T > 0 && max_seqlen >= 1) {
        const size_t need = dsa_attn_fwd_workspace_bytes(T, max_seqlen, 1);
        if (!bitmap || bitmap_bytes < need) return fail(DSA_ERR_WORKSPACE, "selection bitmap: have %zu bytes, need %zu", bitmap_bytes, need);
    }
    return index_topk_impl(q_idx, k_idx, w_idx, cu, T, N, Hi, Di, K, scale, dtype, max_seqlen, idx, n, sel_scores,
                           (uint32_t *)bitmap, ws, ws_bytes, stream);
}

// ---- attention mass of the selected keys (training target of the indexer) ---------------------------
// bitmap + one (T,K) fp32 table per group of kv heads (none when one group takes all kv heads)
extern "C" size_t dsa_attn_mass_workspace_bytes(int T, int N, int Hq, int Hkv, int D, int K, int max_seqlen) {
    if (T <= 0 || N < 0 || Hkv <= 0 || Hq < Hkv || K <= 0) return 0;
    const int g = dsa_mass_groups(Hq, Hkv, D);
    return align_up((size_t)T * bitmap_ldw(max_seqlen) * 4, 256) + (g > 1 ? align_up((size_t)g * T * K * 4, 256) : 0);
}

// saved_bitmap != NULL: the bitmap of idx/n exists already (left by dsa_index_topk_bitmap or a forward) and is only read;
// ws then holds the partial tables alone
static int attn_mass_run(const void *q, const void *k, const float *lse, const int32_t *idx, const int32_t *n, const int32_t *cu,
                         int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale, int dtype, int max_seqlen, float *mass,
                         const void *saved_bitmap, size_t saved_bytes, void *ws, size_t ws_bytes, void *stream) {
    if (int rc = check_attn(T, N, cu, Hq, Hkv, D, K, dtype, idx, n)) return rc;
    if (!q || !k || !lse || !idx || !n || !mass) return fail(DSA_ERR_ARG, "null tensor pointer");
    if (max_seqlen < 1 || max_seqlen > (T > 0 ? T : 1)) return fail(DSA_ERR_ARG, "max_seqlen=%d outside [1,T=%d]", max_seqlen, T);
    if (T == 0) return DSA_OK;
    const int ldw = bitmap_ldw(max_seqlen);
    const size_t bm = align_up((size_t)T * ldw * 4, 256);
    const size_t need = dsa_attn_mass_workspace_bytes(T, N, Hq, Hkv, D, K, max_seqlen) - (saved_bitmap ? bm : 0);
    if (need && (!ws || ws_bytes < need)) return fail(DSA_ERR_WORKSPACE, "mass workspace: have %zu bytes, need %zu", ws_bytes, need);
    if (saved_bitmap && saved_bytes < bm) return fail(DSA_ERR_WORKSPACE, "selection bitmap: have %zu bytes, need %zu", saved_bytes, bm);
    if ((size_t)ldw * 4 > 64 * 1024) return fail(DSA_ERR_UNSUPPORTED, "max_seqlen=%d: selection bitmap row exceeds 64 KiB of LDS", max_seqlen);
    hipStream_t st = (hipStream_t)stream;
    const uint32_t *bitmap = saved_bitmap ? (const uint32_t *)saved_bitmap : (const uint32_t *)ws;
    float *partial = (float *)((char *)ws + (saved_bitmap ? 0 : bm));
    hipError_t e = hipSuccess;
    if (!saved_bitmap) {
        e = dsa_launch_bitmap(idx, n, cu, N, T, K, ldw, (uint32_t *)ws, st);
        if (e != hipSuccess) return hip_fail(e, "bitmap launch");
    }
    e = dsa_launch_tile_mass(q, k, lse, bitmap, ldw, n, cu, N, T, Hq, Hkv, D, K, softmax_scale, partial, mass, st);
    if (e != hipSuccess) return hip_fail(e, "attention mass launch");
    return DSA_OK;
}

extern "C" int dsa_attn_mass(const void *q, const void *k, const float *lse, const int32_t *idx, const int32_t *n,
                             const int32_t *cu, int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale,
                             int dtype, int max_seqlen, float *mass, void *ws, size_t ws_bytes, void *stream) {
    return attn_mass_run(q, k, lse, idx, n, cu, T, N, Hq, Hkv, D, K, softmax_scale, dtype, max_seqlen, mass, nullptr, 0, ws,
                         ws_bytes, stream);
}

extern "C" int dsa_attn_mass_saved_bitmap(const void *q, const void *k, const float *lse, const int32_t *idx, const int32_t *n,
                                          const int32_t *cu, int T, int N, int Hq, int Hkv, int D, int K, float softmax_scale,
                                          int dtype, int max_seqlen, float *mass, const void *bitmap, size_t bitmap_bytes,
                                          void *ws, size_t ws_bytes, void *stream) {
    if (!bitmap) return fail(DSA_ERR_ARG, "null selection bitmap");
    return attn_mass_run(q, k, lse, idx, n, cu, T, N, Hq, Hkv, D, K, softmax_scale, dtype, max_seqlen, mass, bitmap,
                         bitmap_bytes, ws, ws_bytes, stream);
}

// ---- the query-side and the key-side pass of one backward side by side ----
// Both read the same inputs and write different outputs, and a launch of few workgroups ends on its longest walks with
// most CUs idle: the query side then runs on a second stream of the library's own (default priority, one per device,
// made on first use outside any capture) between a fork and a join event, so that to the caller everything still
// happens on the stream it passed.  A stream under capture takes the second one into the capture through the events.
// mode 1 runs the passes side by side for key-side launches of at most this many workgroups (larger ones fill the GPU
// alone) whose work bound T * max_seqlen * Hq * D reaches the second figure (about 0.4 ms of backward: below it the
// fork, the join and the delta pass that the query side otherwise absorbs cost what the overlap gains)
#define DSA_BWD_OVERLAP_MAX_WG (6 * 256)
#define DSA_BWD_OVERLAP_MIN_WORK 6.0e10
struct OverlapCtx {
    hipStream_t aux = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    bool failed = false;
};
static OverlapCtx g_overlap[DSA_MAX_DEVICES];
static std::mutex g_overlap_mu;                          // held from fork to join: the events are shared by every caller
static std::atomic<int> g_bwd_overlap{1};               // 0 never, 1 launches of few workgroups, 2 always
extern "C" int dsa_set_bwd_overlap(int mode) {
    if (mode < 0 || mode > 2) return fail(DSA_ERR_ARG, "bwd overlap mode=%d outside [0,2]", mode);
    g_bwd_overlap.store(mode, std::memory_order_relaxed);
    return DSA_OK;
}
extern "C" int dsa_get_bwd_overlap(void) { return g_bwd_overlap.load(std::memory_order_relaxed); }
// null when the second stream is not to be had (then the passes run one after the other); call with g_overlap_mu held
static OverlapCtx *overlap_ctx(hipStream_t main_stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= DSA_MAX_DEVICES) return nullptr;
    OverlapCtx &c = g_overlap[dev];
    if (c.aux) return &c;
    if (c.failed) return nullptr;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (main_stream && (hipStreamIsCapturing(main_stream, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone)) {
        (void)hipGetLastError();
        return nullptr;                                  // nothing is created while a capture runs
    }
    if (hipStreamCreateWithFlags(&c.aux, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&c.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&c.join, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        c.aux = nullptr;
        c.failed = true;
        return nullptr;
    }
    return &c;
}

// ---- indexer backward: gradients of the selected scores w.r.t. the indexer's inputs --------------------
extern "C" size_t dsa_indexer_bwd_workspace_bytes(int T, int Di, int max_seqlen) {
    if (T <= 0) return 0;
    const int ldw = bitmap_ldw(max_seqlen);                    // selection bitmap + slot prefix table + partial dk sums
    return 2 * align_up((size_t)T * ldw * 4, 256) + align_up(dsa_indexer_bwd_partial_bytes(T, Di, ldw), 256);
}

extern "C" int dsa_indexer_bwd(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *idx, const int32_t *n,
                               const float *dscore, const int32_t *cu, int T, int N, int Hi, int Di, int K, float scale,
                               int dtype, int max_seqlen, void *dq_idx, void *dk_idx, float *dw, void *ws, size_t ws_bytes,
                               void *stream) {
    if (int rc = check_packed(T, N, cu)) return rc;
    if (dtype != DSA_DTYPE_BF16) return fail(DSA_ERR_UNSUPPORTED, "indexer tensors must be bf16 (dtype code %d)", dtype);
    if (Hi < 1 || Hi > 64) return fail(DSA_ERR_UNSUPPORTED, "Hi=%d: 1..64 indexer heads", Hi);
    if (!(Di == 64 || Di == 128)) return fail(DSA_ERR_UNSUPPORTED, "Di=%d: the indexer backward covers 64 and 128", Di);
    if (K < 1) return fail(DSA_ERR_ARG, "top_k=%d must be >= 1", K);
    if (!q_idx || !k_idx || !w_idx || !idx || !n || !dscore || !dq_idx || !dk_idx || !dw) return fail(DSA_ERR_ARG, "null tensor pointer");
    if (max_seqlen < 1 || max_seqlen > (T > 0 ? T : 1)) return fail(DSA_ERR_ARG, "max_seqlen=%d outside [1,T=%d]", max_seqlen, T);
    if (T == 0) return DSA_OK;
    const size_t need = dsa_indexer_bwd_workspace_bytes(T, Di, max_seqlen);
    if (!ws || ws_bytes < need) return fail(DSA_ERR_WORKSPACE, "indexer backward workspace: have %zu bytes, need %zu", ws_bytes, need);
    const int ldw = bitmap_ldw(max_seqlen);
    if ((size_t)ldw * 4 > 64 * 1024) return fail(DSA_ERR_UNSUPPORTED, "max_seqlen=%d: selection bitmap row exceeds 64 KiB of LDS", max_seqlen);
    hipStream_t st = (hipStream_t)stream;
    const size_t bm = align_up((size_t)T * ldw * 4, 256);
    uint32_t *bitmap = (uint32_t *)ws;
    int32_t *prefix = (int32_t *)((char *)ws + bm);
    float *partial = (float *)((char *)ws + 2 * bm);
    hipError_t e = dsa_launch_bitmap(idx, n, cu, N, T, K, ldw, bitmap, st);
    if (e != hipSuccess) return hip_fail(e, "bitmap launch");
    // the query side (dq_idx, dw) and the key side (dk_idx) read the same inputs and write different outputs: side by
    // side on two streams where dsa_set_bwd_overlap allows it, as the two passes of the attention backward
    std::unique_lock<std::mutex> ov_lock;
    OverlapCtx *ov = nullptr;
    const int ov_mode = g_bwd_overlap.load(std::memory_order_relaxed);
    // (mode 1: launches up to 16 384 tokens with T * max_seqlen * Hi * Di of at least 1e10 - 8192 tokens 0.24 -> 0.20 ms,
    // 16 384 tokens 0.53 -> 0.48; at 32 768 tokens both sides fill the GPU alone and nothing is gained)
    if (ov_mode == 2 || (ov_mode == 1 && T <= 16384 && (double)T * max_seqlen * Hi * Di >= 1e10)) {
        ov_lock = std::unique_lock<std::mutex>(g_overlap_mu);
        ov = overlap_ctx(st);
        if (!ov) ov_lock.unlock();
    }
    hipStream_t sq = st;
    if (ov) {
        e = hipEventRecord(ov->fork, st);
        if (e == hipSuccess) e = hipStreamWaitEvent(ov->aux, ov->fork, 0);
        if (e != hipSuccess) return hip_fail(e, "fork to the second stream");
        sq = ov->aux;
    }
    int rc = DSA_OK;
    e = dsa_launch_indexer_bwd(q_idx, k_idx, w_idx, dscore, bitmap, prefix, ldw, cu, N, T, Hi, Di, K, scale, dq_idx, dk_idx, dw,
                               partial, st, sq);
    if (e != hipSuccess) rc = hip_fail(e, "indexer backward launch");
    if (ov) {
        e = hipEventRecord(ov->join, ov->aux);
        if (e == hipSuccess) e = hipStreamWaitEvent(st, ov->join, 0);
        if (e != hipSuccess && rc == DSA_OK) rc = hip_fail(e, "join of the second stream");
    }
    return rc;
}

extern "C" size_t dsa_attn_bwd_workspace_bytes(int T, int Hq, int max_seqlen, int has_idx) {
    if (T <= 0) return 0;
    size_t b = align_up((size_t)T * Hq * 4, 256);                                     // delta
    if (has_idx) b += align_up((size_t)T * bitmap_ldw(max_seqlen) * 4, 256);          // selection bitmap
    b += align_up(dsa_tile_dkv_partial_bytes(T), 256);                                // dK / dV of key-tile walks in pieces
    return b + align_up(dsa_tile_order_bytes(T), 256);                                // launch order of the key tiles
}

extern "C" size_t dsa_attn_bwd_bitmap_offset(int T, int Hq) {
    if (T <= 0 || Hq <= 0) return 0;
    return align_up((size_t)T * Hq * 4, 256);
}

// the backward proper: every buffer named, so that the two entry points below differ only in where the buffers live
static int attn_bwd_run(const void *dout, const void *q, const void *k, const void *v, const void *out, const float *lse,
                        const int32_t *idx, const int32_t *n, const int32_t *cu, int T, int N, int Hq, int Hkv, int D, int K,
                        float softmax_scale, int max_seqlen, int causal, void *dq, void *dk, void *dv, float *delta,
                        uint32_t *bitmap, float *partial, size_t partial_bytes, int32_t *order, int parts, hipStream_t st) {
    const int ldw = bitmap_ldw(max_seqlen);
    if (idx && (size_t)ldw * 4 > 64 * 1024) return fail(DSA_ERR_UNSUPPORTED, "max_seqlen=%d: selection bitmap row exceeds 64 KiB of LDS", max_seqlen);
    const int split = pos_split_for(idx, K);
    hipError_t e = hipSuccess;
    // the two passes side by side on two streams: launches of few workgroups only (larger ones fill the GPU alone)
    std::unique_lock<std::mutex> ov_lock;
    OverlapCtx *ov = nullptr;
    const int ov_mode = g_bwd_overlap.load(std::memory_order_relaxed);
    if ((parts & DSA_BWD_DQ) && (parts & DSA_BWD_DKV) && ov_mode > 0) {
        const int64_t dkv_wg = ((int64_t)T / 128 + N) * Hkv * (D > 128 ? 2 : 1);
        const double work = (double)T * max_seqlen * Hq * D;
        if (ov_mode == 2 || (dkv_wg <= DSA_BWD_OVERLAP_MAX_WG && work >= DSA_BWD_OVERLAP_MIN_WORK)) {
            ov_lock = std::unique_lock<std::mutex>(g_overlap_mu);
            ov = overlap_ctx(st);
            if (!ov) ov_lock.unlock();
        }
    }
    // delta = rowsum(dO * O): a pass of its own, unless the tile dQ kernel of the same call owns every query row
    // (no row beyond the tile/gather split) - then that kernel forms it from the dO rows it loads anyway - and the
    // key side, which reads every delta, runs after it
    const bool fuse_delta = (parts & DSA_BWD_DELTA) && (parts & DSA_BWD_DQ) && split > 0 && max_seqlen <= split && !ov;
    if ((parts & DSA_BWD_DELTA) && !fuse_delta) {
        e = dsa_launch_delta(dout, out, T, Hq, D, delta, st);
        if (e != hipSuccess) return hip_fail(e, "delta launch");
    }
    if ((parts & DSA_BWD_BITMAP) && idx) {
        e = dsa_launch_bitmap(idx, n, cu, N, T, K, ldw, bitmap, st);
        if (e != hipSuccess) return hip_fail(e, "bitmap launch");
    }
    hipStream_t sq = st;
    if (ov) {
        e = hipEventRecord(ov->fork, st);
        if (e == hipSuccess) e = hipStreamWaitEvent(ov->aux, ov->fork, 0);
        if (e != hipSuccess) return hip_fail(e, "fork to the second stream");
        sq = ov->aux;
    }
    int rc = DSA_OK;
    // (side by side, the key side is issued first: it is the longer pass and starts with its longest walks)
    if (ov) {
        e = dsa_launch_tile_dkv(dout, q, k, v, lse, delta, bitmap, ldw, cu, N, T, Hq, Hkv, D, softmax_scale, causal, order, partial,
                                partial_bytes, dk, dv, st);
        if (e != hipSuccess) rc = hip_fail(e, "tile dkv launch");
    }
    if (rc == DSA_OK && (parts & DSA_BWD_DQ)) {
        if (split > 0) {
            e = dsa_launch_tile_dq(dout, q, k, v, lse, delta, bitmap, ldw, cu, N, T, Hq, Hkv, D, softmax_scale, split, causal, dq,
                                   fuse_delta ? out : nullptr, delta, sq);
            if (e != hipSuccess) rc = hip_fail(e, "tile dq launch");
        }
        if (rc == DSA_OK && max_seqlen > split) {
            e = dsa_launch_gather_dq(dout, q, k, v, lse, delta, idx, n, cu, N, T, Hq, Hkv, D, K, softmax_scale, split, dq, sq);
            if (e != hipSuccess) rc = hip_fail(e, "gather dq launch");
        }
    }
    if (rc == DSA_OK && !ov && (parts & DSA_BWD_DKV)) {
        e = dsa_launch_tile_dkv(dout, q, k, v, lse, delta, bitmap, ldw, cu, N, T, Hq, Hkv, D, softmax_scale, causal, order, partial,
                                partial_bytes, dk, dv, st);
        if (e != hipSuccess) rc = hip_fail(e, "tile dkv launch");
    }
    if (ov) {                                            // joined also after a failed launch: the caller's stream stays whole
        e = hipEventRecord(ov->join, ov->aux);
        if (e == hipSuccess) e = hipStreamWaitEvent(st, ov->join, 0);
        if (e != hipSuccess && rc == DSA_OK) rc = hip_fail(e, "join of the second stream");
    }
    return rc;
}

static int check_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out, const float *lse,
                     const int32_t *idx, const int32_t *n, const int32_t *cu, int T, int N, int Hq, int Hkv, int D, int K,
                     int dtype, int max_seqlen, int causal, const void *dq, const void *dk, const void *dv) {
    if (int rc = check_attn(T, N, cu, Hq, Hkv, D, K, dtype, idx, n)) return rc;
    if (!causal && idx) return fail(DSA_ERR_ARG, "a key selection (idx) implies causal attention");
    if (!dout || !q || !k || !v || !out || !lse || !dq || !dk || !dv) return fail(DSA_ERR_ARG, "null tensor pointer");
    if (max_seqlen < 1 || max_seqlen > (T > 0 ? T : 1)) return fail(DSA_ERR_ARG, "max_seqlen=%d outside [1,T=%d]", max_seqlen, T);
    return DSA_OK;
}

extern "C" int dsa_attn_bwd_parts(const void *dout, const void *q, const void *k, const void *v, const void *out,
                                  const float *lse, const int32_t *idx, const int32_t *n, const int32_t *cu, int T,
                                  int N, int Hq, int Hkv, int D, int K, float softmax_scale, int dtype, int max_seqlen,
                                  int causal, void *dq, void *dk, void *dv, void *ws, size_t ws_bytes, int parts,
                                  void *stream) {
    if (int rc = check_bwd(dout, q, k, v, out, lse, idx, n, cu, T, N, Hq, Hkv, D, K, dtype, max_seqlen, causal, dq, dk, dv)) return rc;
    if (T == 0) return DSA_OK;
    const size_t need = dsa_attn_bwd_workspace_bytes(T, Hq, max_seqlen, idx != nullptr);
    if (!ws || ws_bytes < need) return fail(DSA_ERR_WORKSPACE, "backward workspace: have %zu bytes, need %zu", ws_bytes, need);
    float *delta = (float *)ws;
    uint32_t *bitmap = idx ? (uint32_t *)((char *)ws + dsa_attn_bwd_bitmap_offset(T, Hq)) : nullptr;
    int32_t *order = (int32_t *)((char *)ws + need - align_up(dsa_tile_order_bytes(T), 256));
    const size_t partial_bytes = dsa_tile_dkv_partial_bytes(T);
    float *partial = partial_bytes ? (float *)((char *)order - align_up(partial_bytes, 256)) : nullptr;
    return attn_bwd_run(dout, q, k, v, out, lse, idx, n, cu, T, N, Hq, Hkv, D, K, softmax_scale, max_seqlen, causal, dq, dk, dv,
                        delta, bitmap, partial, partial_bytes, order, parts, (hipStream_t)stream);
}

// Scratch of the backward that nothing outlives: delta, the launch order of the key tiles and - only for launches small
// enough to be cut into pieces (at most 1024 workgroups before the cut) - the fp32 partial sums of those pieces.
static size_t bwd_partial_bytes_for(int T, int N, int Hkv, int D) {
    const int64_t wg_per_tile = (int64_t)Hkv * (D > 128 ? 2 : 1);
    if (((int64_t)T / 128 + N) * wg_per_tile > 4 * 256) return 0;
    return dsa_tile_dkv_partial_bytes(T);
}
extern "C" size_t dsa_attn_bwd_scratch_bytes(int T, int N, int Hq, int Hkv, int D) {
    if (T <= 0 || N < 0 || Hq <= 0 || Hkv <= 0) return 0;
    return align_up((size_t)T * Hq * 4, 256) + align_up(bwd_partial_bytes_for(T, N, Hkv, D), 256) +
           align_up(dsa_tile_order_bytes(T), 256);
}

extern "C" int dsa_attn_bwd_saved_bitmap(const void *dout, const void *q, const void *k, const void *v, const void *out,
                                         const float *lse, const int32_t *idx, const int32_t *n, const int32_t *cu, int T,
                                         int N, int Hq, int Hkv, int D, int K, float softmax_scale, int dtype,
                                         int max_seqlen, int causal, void *dq, void *dk, void *dv, const void *fwd_ws,
                                         size_t fwd_ws_bytes, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_bwd(dout, q, k, v, out, lse, idx, n, cu, T, N, Hq, Hkv, D, K, dtype, max_seqlen, causal, dq, dk, dv)) return rc;
    if (T == 0) return DSA_OK;
    if (idx) {
        if (pos_split_for(idx, K) <= 0) return fail(DSA_ERR_ARG, "with the tile crossover at 0 the forward builds no bitmap: use dsa_attn_bwd");
        const size_t have = dsa_attn_fwd_workspace_bytes(T, max_seqlen, 1);
        if (!fwd_ws || fwd_ws_bytes < have) return fail(DSA_ERR_WORKSPACE, "forward workspace (selection bitmap): have %zu bytes, need %zu", fwd_ws_bytes, have);
    }
    const size_t need = dsa_attn_bwd_scratch_bytes(T, N, Hq, Hkv, D);
    if (!scratch || scratch_bytes < need) return fail(DSA_ERR_WORKSPACE, "backward scratch: have %zu bytes, need %zu", scratch_bytes, need);
    float *delta = (float *)scratch;
    const size_t partial_bytes = bwd_partial_bytes_for(T, N, Hkv, D);
    float *partial = partial_bytes ? (float *)((char *)scratch + align_up((size_t)T * Hq * 4, 256)) : nullptr;
    int32_t *order = (int32_t *)((char *)scratch + need - align_up(dsa_tile_order_bytes(T), 256));
    // the kernels only read the bitmap; the forward's workspace is not written here
    uint32_t *bitmap = idx ? const_cast<uint32_t *>((const uint32_t *)fwd_ws) : nullptr;
    return attn_bwd_run(dout, q, k, v, out, lse, idx, n, cu, T, N, Hq, Hkv, D, K, softmax_scale, max_seqlen, causal, dq, dk, dv,
                        delta, bitmap, partial, partial_bytes, order, DSA_BWD_ALL & ~DSA_BWD_BITMAP, (hipStream_t)stream);
}

extern "C" int dsa_attn_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out,
                            const float *lse, const int32_t *idx, const int32_t *n, const int32_t *cu, int T, int N,
                            int Hq, int Hkv, int D, int K, float softmax_scale, int dtype, int max_seqlen, int causal,
                            void *dq, void *dk, void *dv, void *ws, size_t ws_bytes, void *stream) {
    return dsa_attn_bwd_parts(dout, q, k, v, out, lse, idx, n, cu, T, N, Hq, Hkv, D, K, softmax_scale, dtype, max_seqlen,
                              causal, dq, dk, dv, ws, ws_bytes, DSA_BWD_ALL, stream);
}

extern "C" int dsa_dense_fwd(const void *q, const void *k, const void *v, const int32_t *cu, int T, int N, int Hq, int Hkv,
                             int D, float softmax_scale, int dtype, int max_seqlen, int causal, void *out, float *lse,
                             void *stream) {
    return dsa_attn_fwd(q, k, v, nullptr, nullptr, cu, T, N, Hq, Hkv, D, 0, softmax_scale, dtype, max_seqlen, causal, out, lse,
                        nullptr, 0, stream);
}

extern "C" int dsa_dense_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out, const float *lse,
                             const int32_t *cu, int T, int N, int Hq, int Hkv, int D, float softmax_scale, int dtype,
                             int max_seqlen, int causal, void *dq, void *dk, void *dv, void *ws, size_t ws_bytes,
                             void *stream) {
    return dsa_attn_bwd(dout, q, k, v, out, lse, nullptr, nullptr, cu, T, N, Hq, Hkv, D, 0, softmax_scale, dtype, max_seqlen,
                        causal, dq, dk, dv, ws, ws_bytes, stream);
}

// ---------------------------------------------------------------------------------------------------
// prologue / gate
// ---------------------------------------------------------------------------------------------------
static int check_prologue(int T, int Hq, int Hkv, int D, int R, int cs_dtype, int64_t q_head, int64_t k_head) {
    if (T < 0 || Hq < 1 || Hkv < 1) return fail(DSA_ERR_ARG, "T=%d Hq=%d Hkv=%d", T, Hq, Hkv);
    if (!(D == 64 || D == 128 || D == 256)) return fail(DSA_ERR_UNSUPPORTED, "head_dim=%d: need 64, 128 or 256", D);
    if (R < 0 || R > D || R % 16) return fail(DSA_ERR_UNSUPPORTED, "rotary width R=%d: need a multiple of 16 up to head_dim=%d", R, D);
    if (cs_dtype != DSA_DTYPE_BF16 && cs_dtype != DSA_DTYPE_FP32) return fail(DSA_ERR_ARG, "cos/sin dtype code %d", cs_dtype);
    if (q_head % 8 || k_head % 8) return fail(DSA_ERR_ARG, "head strides must be multiples of 8 elements (16-byte rows)");
    return DSA_OK;
}

extern "C" size_t dsa_qk_norm_rope_bwd_workspace_bytes(int T, int D) {
    if (T <= 0 || D <= 0) return 0;
    return (size_t)dsa_prologue_bwd_blocks(T) * 2 * D * sizeof(float);
}

extern "C" int dsa_qk_norm_rope_fwd(const void *q_in, int64_t q_tok, int64_t q_head, const void *k_in, int64_t k_tok,
                                    int64_t k_head, const void *qw, const void *kw, float eps, int norm_flags,
                                    const void *cosp, const void *sinp, int cs_dtype, int R, int T, int Hq, int Hkv, int D,
                                    void *q_out, void *k_out, float *q_rstd, float *k_rstd, void *stream) {
    if (int rc = check_prologue(T, Hq, Hkv, D, R, cs_dtype, q_head, k_head)) return rc;
    if (!q_in || !k_in || !qw || !kw || !q_out || !k_out || !q_rstd || !k_rstd || (R > 0 && (!cosp || !sinp)))
        return fail(DSA_ERR_ARG, "null tensor pointer");
    if (q_tok % 8 || k_tok % 8) return fail(DSA_ERR_ARG, "token strides must be multiples of 8 elements");
    hipError_t e = dsa_launch_qk_norm_rope_fwd(q_in, q_tok, q_head, k_in, k_tok, k_head, qw, kw, (norm_flags & DSA_NORM_WEIGHT_BF16) != 0, eps,
                                               (norm_flags & DSA_NORM_OFFSET) ? 1.f : 0.f,
                                               cosp, sinp, cs_dtype == DSA_DTYPE_FP32, R, T, Hq, Hkv, D, q_out, k_out, q_rstd,
                                               k_rstd, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "qk_norm_rope forward launch");
}

extern "C" int dsa_qk_norm_rope_bwd(const void *gq, const void *gk, const void *q_in, int64_t q_tok, int64_t q_head,
                                    const void *k_in, int64_t k_tok, int64_t k_head, const void *qw, const void *kw,
                                    int norm_flags, const void *cosp, const void *sinp, int cs_dtype, int R,
                                    const float *q_rstd, const float *k_rstd, int T, int Hq, int Hkv, int D, void *dq_in,
                                    int64_t dq_tok, int64_t dq_head, void *dk_in, int64_t dk_tok, int64_t dk_head,
                                    float *dqw, float *dkw, void *ws, size_t ws_bytes, void *stream) {
    if (int rc = check_prologue(T, Hq, Hkv, D, R, cs_dtype, q_head, k_head)) return rc;
    if (!gq || !gk || !q_in || !k_in || !qw || !kw || !q_rstd || !k_rstd || !dq_in || !dk_in || !dqw || !dkw ||
        (R > 0 && (!cosp || !sinp)))
        return fail(DSA_ERR_ARG, "null tensor pointer");
    if (q_tok % 8 || k_tok % 8 || dq_tok % 8 || dk_tok % 8 || dq_head % 8 || dk_head % 8)
        return fail(DSA_ERR_ARG, "strides must be multiples of 8 elements");
    const size_t need = dsa_qk_norm_rope_bwd_workspace_bytes(T, D);
    if (need && (!ws || ws_bytes < need)) return fail(DSA_ERR_WORKSPACE, "prologue backward workspace: have %zu bytes, need %zu", ws_bytes, need);
    hipError_t e = dsa_launch_qk_norm_rope_bwd(gq, gk, q_in, q_tok, q_head, k_in, k_tok, k_head, qw, kw, (norm_flags & DSA_NORM_WEIGHT_BF16) != 0,
                                               (norm_flags & DSA_NORM_OFFSET) ? 1.f : 0.f,
                                               cosp, sinp, cs_dtype == DSA_DTYPE_FP32, R, q_rstd, k_rstd, T, Hq, Hkv, D, dq_in,
                                               dq_tok, dq_head, dk_in, dk_tok, dk_head, dqw, dkw, (float *)ws,
                                               (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "qk_norm_rope backward launch");
}

extern "C" int dsa_sigmoid_gate_fwd(const void *x, const void *gate, int64_t gate_tok, int64_t gate_head, int T, int H, int D,
                                    void *y, void *stream) {
    if (T < 0 || H < 1 || D < 8 || D % 8 || gate_tok % 8 || gate_head % 8) return fail(DSA_ERR_ARG, "T=%d H=%d D=%d or strides not multiples of 8", T, H, D);
    if (!x || !gate || !y) return fail(DSA_ERR_ARG, "null tensor pointer");
    hipError_t e = dsa_launch_sigmoid_gate_fwd(x, gate, gate_tok, gate_head, D, H, T, y, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "sigmoid gate forward launch");
}

extern "C" int dsa_sigmoid_gate_bwd(const void *gy, const void *x, const void *gate, int64_t gate_tok, int64_t gate_head,
                                    int T, int H, int D, void *dx, void *dgate, int64_t dgate_tok, int64_t dgate_head,
                                    void *stream) {
    if (T < 0 || H < 1 || D < 8 || D % 8 || gate_tok % 8 || gate_head % 8 || dgate_tok % 8 || dgate_head % 8)
        return fail(DSA_ERR_ARG, "T=%d H=%d D=%d or strides not multiples of 8", T, H, D);
    if (!gy || !x || !gate || !dx || !dgate) return fail(DSA_ERR_ARG, "null tensor pointer");
    hipError_t e = dsa_launch_sigmoid_gate_bwd(gy, x, gate, gate_tok, gate_head, D, H, T, dx, dgate, dgate_tok, dgate_head,
                                               (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "sigmoid gate backward launch");
}

// ---- fp32 operands carried as stacked split-bf16 rows (the host operator's fp32 path for head_dim <= 64) ----
extern "C" int dsa_split_bf16_stack(const float *x, int64_t rows, int D, int order, void *y, void *stream) {
    if (rows < 0 || D < 4 || D % 4 || (order != 0 && order != 1)) return fail(DSA_ERR_ARG, "rows=%lld D=%d order=%d", (long long)rows, D, order);
    if (rows > 0 && (!x || !y)) return fail(DSA_ERR_ARG, "null tensor pointer");
    hipError_t e = dsa_launch_split_stack(x, rows, D, order, y, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "split/stack launch");
}
extern "C" int dsa_split_bf16_combine(const void *y, int64_t rows, int D, int part, float *out, void *stream) {
    if (rows < 0 || D < 4 || D % 4 || part < 1 || part > 3) return fail(DSA_ERR_ARG, "rows=%lld D=%d part=%d", (long long)rows, D, part);
    if (rows > 0 && (!y || !out)) return fail(DSA_ERR_ARG, "null tensor pointer");
    hipError_t e = dsa_launch_split_combine(y, rows, D, part, out, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "split/combine launch");
}
extern "C" int dsa_split_bf16_stack_qkv(const float *q, const float *k, const float *v, int64_t rows_q, int64_t rows_kv, int D,
                                        void *yq, void *yk, void *yv, void *stream) {
    if (rows_q < 0 || rows_kv < 0 || D < 4 || D % 4) return fail(DSA_ERR_ARG, "rows_q=%lld rows_kv=%lld D=%d", (long long)rows_q, (long long)rows_kv, D);
    if ((rows_q > 0 && (!q || !yq)) || (rows_kv > 0 && (!k || !v || !yk || !yv))) return fail(DSA_ERR_ARG, "null tensor pointer");
    hipError_t e = dsa_launch_split_stack_qkv(q, k, v, rows_q, rows_kv, D, yq, yk, yv, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "split/stack launch");
}
extern "C" int dsa_split_bf16_combine_qkv(const void *yq, const void *yk, const void *yv, int64_t rows_q, int64_t rows_kv, int D,
                                          float *dq, float *dk, float *dv, void *stream) {
    if (rows_q < 0 || rows_kv < 0 || D < 4 || D % 4) return fail(DSA_ERR_ARG, "rows_q=%lld rows_kv=%lld D=%d", (long long)rows_q, (long long)rows_kv, D);
    if ((rows_q > 0 && (!yq || !dq)) || (rows_kv > 0 && (!yk || !yv || !dk || !dv))) return fail(DSA_ERR_ARG, "null tensor pointer");
    hipError_t e = dsa_launch_split_combine_qkv(yq, yk, yv, rows_q, rows_kv, D, dq, dk, dv, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "split/combine launch");
}

// ---- three fp32 arrays rounded to bf16 by one launch (the indexer's inputs of an fp32 caller) ----
extern "C" int dsa_round_bf16_x3(const float *a, const float *b, const float *c, int64_t na, int64_t nb, int64_t nc, void *ya,
                                 void *yb, void *yc, void *stream) {
    if (na < 0 || nb < 0 || nc < 0) return fail(DSA_ERR_ARG, "negative element count");
    if ((na > 0 && (!a || !ya)) || (nb > 0 && (!b || !yb)) || (nc > 0 && (!c || !yc))) return fail(DSA_ERR_ARG, "null tensor pointer");
    if ((((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15) || (((uintptr_t)ya | (uintptr_t)yb | (uintptr_t)yc) & 7))
        return fail(DSA_ERR_ARG, "inputs must be 16-byte aligned, outputs 8-byte aligned");
    hipError_t e = dsa_launch_round_bf16_x3(a, b, c, na, nb, nc, ya, yb, yc, (hipStream_t)stream);
    return e == hipSuccess ? DSA_OK : hip_fail(e, "bf16 rounding launch");
}
