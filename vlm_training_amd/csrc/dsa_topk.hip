// Stage D2: per-query top-k over one row of fp32 scores, total order (score descending, column
// ascending).  One 256-thread workgroup per query row.
//
//   1. rows with pos+1 <= K are the whole causal window: write the range, done;
//   2. MSB-first radix select (3 passes of 11, 11 and 10 bits) over order-preserving uint32 keys finds the
//      K-th largest key tau and how many keys equal to tau are still wanted (need_eq); the first histogram
//      is filled while the row is read;
//   3. an index-ordered compaction keeps key > tau, plus the first need_eq keys == tau.  The row is
//      split into four contiguous quarters (one per wave); per-quarter counts give every wave its
//      output offset, so the result comes out ascending and deterministic without sorting.
//
// Rows up to TOPK_LDS_CAP keys are read from HBM once and kept in LDS as keys.
// With a sel_out pointer the kernel also writes the scores of the selected keys beside their indices (the key it ranks
// by is the score, bit for bit, but for the sign of a zero).
//
// With a bitmap pointer the kernel also leaves the row's inverted selection (bit c of the row's ldw words = "key column c
// of the segment is selected", what dsa_bitmap_kernel builds from the finished list): the compaction's ballots are those
// words already, so the list need not be read back.
#include "dsa_common.h"

#define TOPK_THREADS 256
#define TOPK_LDS_CAP 8192
#define TOPK_BINS 2048                                  // 11-bit digits (the last pass uses 1024 of them)

// the score a key stands for (-0.0 comes back as +0.0: score_key folds the two)
__device__ __forceinline__ float key_score(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
__device__ __forceinline__ uint32_t score_key(float x) {
    uint32_t u = __float_as_uint(x);
    if (u == 0x80000000u) u = 0u;                       // -0.0 ties with +0.0
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // larger float <=> larger key
}

// `only`: 0 = every row of the launch; 1 = rows of at most lds_keys keys (the others belong to a second launch of the
// uncached kernel); 2 = rows longer than skip_upto keys.  A launch whose bound on the longest row exceeds the LDS cache
// is split this way, so that the rows that do fit are still read from HBM once - the bound may be far above the real
// longest row (max_seqlen = the packed length when the caller holds no better one).
template <bool CACHED>
__global__ __launch_bounds__(TOPK_THREADS) void dsa_topk_rows_kernel(
    const float *__restrict__ scores, int64_t ld, int row_begin, const int32_t *__restrict__ cu, int N, int K, int lds_keys,
    int only, int skip_upto, int32_t *__restrict__ idx_out, int32_t *__restrict__ n_out, uint32_t *__restrict__ bitmap,
    int ldw, float *__restrict__ sel_out) {
    __shared__ uint32_t hist[TOPK_BINS];
    __shared__ uint32_t wave_tot[4];
    __shared__ uint32_t sel_digit, sel_remaining;
    __shared__ uint32_t cnt_gt[4], cnt_eq[4];
    extern __shared__ __attribute__((aligned(16))) uint32_t keys_lds[];   // CACHED: the launch's longest row; the fewer bytes, the more rows per CU

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int t = row_begin + blockIdx.x;
    const int seg = find_segment(cu, N, t);
    const int s0 = cu[seg];
    // a row never reaches past its ld columns: with a max_seqlen below the longest segment (a caller's mistake) the
    // selection of the long rows is wrong, but nothing outside the score rows is read
    const int nvalid = (int)min((int64_t)(t - s0 + 1), ld);
    int32_t *orow = idx_out + (int64_t)t * K;
    if (only == 1 && nvalid > lds_keys) return;
    if (only == 2 && nvalid <= skip_upto) return;

    uint32_t *brow = bitmap ? bitmap + (int64_t)t * ldw : nullptr;
    float *srow = sel_out ? sel_out + (int64_t)t * K : nullptr;   // the scores of the selected keys, slot by slot (0 past n)
    const float *row = scores + (int64_t)(t - row_begin) * ld;
    if (nvalid <= K) {
        for (int i = tid; i < K; i += TOPK_THREADS) orow[i] = (i < nvalid) ? (s0 + i) : -1;
        if (srow)
            for (int i = tid; i < K; i += TOPK_THREADS) srow[i] = (i < nvalid) ? row[i] : 0.f;
        if (tid == 0) n_out[t] = nvalid;
        if (brow)
            for (int w = tid; w < ldw; w += TOPK_THREADS) {
                const int left = nvalid - 32 * w;       // columns of this word inside the window
                brow[w] = left >= 32 ? ~0u : (left > 0 ? (1u << left) - 1u : 0u);
            }
        return;
    }
    const bool cached = CACHED && nvalid <= lds_keys;    // a row beyond the stated longest one is read from memory each pass
    for (int i = tid; i < TOPK_BINS; i += TOPK_THREADS) hist[i] = 0u;
    __syncthreads();
    if (cached) {
        // 16-byte loads, four per thread in flight: one load per loop iteration would pay the memory latency
        // nvalid / 256 times over
        const float4 *row4 = reinterpret_cast<const float4 *>(row);
        const int n4 = (reinterpret_cast<uintptr_t>(row) & 15) ? 0 : nvalid >> 2;   // a caller's own rows may not be aligned
        for (int base = 0; base < n4; base += 4 * TOPK_THREADS) {
            float4 x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i4 = base + u * TOPK_THREADS + tid;
                x[u] = row4[min(i4, n4 - 1)];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i4 = base + u * TOPK_THREADS + tid;
                if (i4 < n4) {
                    const uint4 kk = {score_key(x[u].x), score_key(x[u].y), score_key(x[u].z), score_key(x[u].w)};
                    *reinterpret_cast<uint4 *>(&keys_lds[4 * i4]) = kk;
                    atomicAdd(&hist[kk.x >> 21], 1u);    // first digit: the top 11 bits
                    atomicAdd(&hist[kk.y >> 21], 1u);
                    atomicAdd(&hist[kk.z >> 21], 1u);
                    atomicAdd(&hist[kk.w >> 21], 1u);
                }
            }
        }
        for (int i = (n4 << 2) + tid; i < nvalid; i += TOPK_THREADS) {
            const uint32_t key = score_key(row[i]);
            keys_lds[i] = key;
            atomicAdd(&hist[key >> 21], 1u);
        }
    }
    auto key_at = [&](int i) -> uint32_t { return cached ? keys_lds[i] : score_key(row[i]); };

    uint32_t prefix = 0u, pmask = 0u, remaining = (uint32_t)K;
    for (int pass = 0; pass < 3; ++pass) {
        const int shift = pass == 0 ? 21 : (pass == 1 ? 10 : 0);
        const uint32_t dmask = pass == 2 ? 1023u : 2047u;
        const int per = pass == 2 ? 4 : 8;              // consecutive digits per thread
        if (pass > 0 || !cached) {
            if (pass > 0) {
                for (int i = tid; i < TOPK_BINS; i += TOPK_THREADS) hist[i] = 0u;
                __syncthreads();
            }
            // eight keys per thread in flight (rows that are not cached come from memory on every sweep)
            for (int base = tid; base < nvalid; base += 8 * TOPK_THREADS) {
                uint32_t kk[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) kk[u] = key_at(min(base + u * TOPK_THREADS, nvalid - 1));
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (base + u * TOPK_THREADS < nvalid && (kk[u] & pmask) == prefix) atomicAdd(&hist[(kk[u] >> shift) & dmask], 1u);
            }
        }
        __syncthreads();
        // thread tid owns the digits [per*tid, per*tid + per); inclusive suffix sum over threads (largest digits first)
        uint32_t own[8], h = 0u;
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            own[b] = b < per ? hist[per * tid + b] : 0u;
            h += own[b];
        }
        uint32_t v = h;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            uint32_t u = __shfl_down(v, off, 64);
            if (lane + off < 64) v += u;
        }
        if (lane == 0) wave_tot[wv] = v;
        __syncthreads();
        for (int w2 = wv + 1; w2 < 4; ++w2) v += wave_tot[w2];
        uint32_t above = v - h;                         // keys with a digit beyond this thread's
        if (above < remaining && remaining <= v) {      // exactly one thread satisfies this; walk its digits from the top
#pragma unroll
            for (int b = 7; b >= 0; --b) {
                if (b < per && above < remaining) {
                    if (remaining <= above + own[b]) {
                        sel_digit = (uint32_t)(per * tid + b);
                        sel_remaining = remaining - above;
                    }
                    above += own[b];
                }
            }
        }
        __syncthreads();
        prefix |= sel_digit << shift;
        pmask |= dmask << shift;
        remaining = sel_remaining;
        __syncthreads();
    }
    const uint32_t tau = prefix, need_eq = remaining;

    // contiguous quarter of the row per wave, multiple of 64 columns
    const int per = (((nvalid + 3) >> 2) + 63) & ~63;
    const int c_begin = min(wv * per, nvalid), c_end = min(c_begin + per, nvalid);
    uint32_t g = 0, e = 0;
    for (int base = c_begin + lane; base < c_end; base += 8 * 64) {
        uint32_t kk[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) kk[u] = key_at(min(base + u * 64, nvalid - 1));
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (base + u * 64 < c_end) {
                g += kk[u] > tau;
                e += kk[u] == tau;
            }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        g += __shfl_xor(g, off, 64);
        e += __shfl_xor(e, off, 64);
    }
    if (lane == 0) { cnt_gt[wv] = g; cnt_eq[wv] = e; }
    __syncthreads();
    uint32_t eq_seen = 0, out_pos = 0;
    for (int w2 = 0; w2 < wv; ++w2) {
        uint32_t eq_take = need_eq > eq_seen ? min(need_eq - eq_seen, cnt_eq[w2]) : 0u;
        out_pos += cnt_gt[w2] + eq_take;
        eq_seen += cnt_eq[w2];
    }
    const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int base = c_begin; base < c_end; base += 4 * 64) {
        uint32_t kk[4];                                 // four chunks of 64 columns fetched, then ranked in index order
#pragma unroll
        for (int u = 0; u < 4; ++u) kk[u] = key_at(min(base + u * 64 + lane, nvalid - 1));
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = base + u * 64 + lane;
            if (base + u * 64 >= c_end) break;          // wave-uniform
            const bool is_gt = i < c_end && kk[u] > tau, is_eq = i < c_end && kk[u] == tau;
            const uint64_t b_eq = __ballot(is_eq);
            const uint32_t eq_rank = eq_seen + (uint32_t)__popcll(b_eq & lt_mask);
            const bool take = is_gt || (is_eq && eq_rank < need_eq);
            const uint64_t b_take = __ballot(take);
            // exactly K keys are taken when every score orders (the radix passes count them); NaN scores can break the
            // count, hence the bound on the slot
            const uint32_t slot = out_pos + (uint32_t)__popcll(b_take & lt_mask);
            if (take && slot < (uint32_t)K) {
                orow[slot] = s0 + i;
                if (srow) srow[slot] = key_score(kk[u]);
            }
            if (brow && lane < 2) {                     // the ballot is the two bitmap words of these 64 columns
                const int w = ((base + u * 64) >> 5) + lane;
                if (w < ldw) brow[w] = (uint32_t)(b_take >> (32 * lane));
            }
            out_pos += (uint32_t)__popcll(b_take);
            eq_seen += (uint32_t)__popcll(b_eq);
        }
    }
    if (brow)                                           // the words behind the window: the quarters end on 64 columns
        for (int w = 2 * ((nvalid + 63) >> 6) + tid; w < ldw; w += TOPK_THREADS) brow[w] = 0u;
    if (tid == 0) n_out[t] = K;
}

extern "C" hipError_t dsa_launch_topk(const float *scores, int64_t ld, int row_begin, int row_end,
                                      const int32_t *cu, int N, int K, int max_row, int32_t *idx, int32_t *n,
                                      uint32_t *bitmap, int ldw, float *sel, hipStream_t stream) {
    const int rows = row_end - row_begin;
    if (rows <= 0) return hipSuccess;
    if (max_row <= TOPK_LDS_CAP) {
        hipLaunchKernelGGL(dsa_topk_rows_kernel<true>, dim3(rows), dim3(TOPK_THREADS), (size_t)((max_row + 3) & ~3) * 4, stream,
                           scores, ld, row_begin, cu, N, K, (max_row + 3) & ~3, 0, 0, idx, n, bitmap, ldw, sel);
    } else {
        hipLaunchKernelGGL(dsa_topk_rows_kernel<true>, dim3(rows), dim3(TOPK_THREADS), (size_t)TOPK_LDS_CAP * 4, stream, scores,
                           ld, row_begin, cu, N, K, TOPK_LDS_CAP, 1, 0, idx, n, bitmap, ldw, sel);
        hipLaunchKernelGGL(dsa_topk_rows_kernel<false>, dim3(rows), dim3(TOPK_THREADS), 16, stream, scores, ld, row_begin, cu,
                           N, K, 0, 2, TOPK_LDS_CAP, idx, n, bitmap, ldw, sel);
    }
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// The KL divergence of the indexer's distribution over the selected keys (their scores sel[t,j], 0 for j >= n[t], come
// out of the selection kernel's compaction) from a target distribution (the attention mass), with its gradient w.r.t.
// the scores.
// ------------------------------------------------------------------------------------------------

// block-wide reductions over 256 threads (4 waves)
__device__ __forceinline__ float block_max_256(float v, float *red) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}
__device__ __forceinline__ float block_sum_256(float v, float *red) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}
// One workgroup per query row.  loss[t] = sum_j p_j (log p_j - log softmax(I)_j) over j < n[t] (terms with p_j = 0
// are 0), dscore[t,j] = (softmax(I)_j - p_j) * grad_scale, 0 for j >= n[t].
__global__ __launch_bounds__(256) void dsa_indexer_kl_kernel(const float *__restrict__ sel, const float *__restrict__ mass,
                                                              const int32_t *__restrict__ nsel, int K, float grad_scale,
                                                              float *__restrict__ loss, float *__restrict__ dscore) {
    __shared__ float red[4];
    const int t = blockIdx.x, nt = nsel[t];
    const float *irow = sel + (int64_t)t * K, *prow = mass + (int64_t)t * K;
    float m = -INFINITY;
    for (int j = threadIdx.x; j < nt; j += 256) m = fmaxf(m, irow[j]);
    m = block_max_256(m, red);
    float z = 0.f;
    for (int j = threadIdx.x; j < nt; j += 256) z += __expf(irow[j] - m);
    z = block_sum_256(z, red);
    const float lse = m + __logf(z);
    float acc = 0.f;
    for (int j = threadIdx.x; j < K; j += 256) {
        float g = 0.f;
        if (j < nt) {
            const float p = prow[j], logq = irow[j] - lse;
            if (p > 0.f) acc += p * (__logf(p) - logq);
            g = (__expf(logq) - p) * grad_scale;
        }
        if (dscore) dscore[(int64_t)t * K + j] = g;
    }
    acc = block_sum_256(acc, red);
    if (threadIdx.x == 0) loss[t] = nt > 0 ? acc : 0.f;
}

// The same for rows of at most 256 * NV scores (K a multiple of 4, rows 16-byte aligned): one wave per row, the row read
// once with all its 16-byte loads in flight and held in registers, reductions inside the wave - no pass over the row
// waits for another and no barrier (the kernel above reads the scores three times and meets at three barriers).
template <int NV>
__global__ __launch_bounds__(256) void dsa_indexer_kl_rows_kernel(const float *__restrict__ sel, const float *__restrict__ mass,
                                                                   const int32_t *__restrict__ nsel, int T, int K,
                                                                   float grad_scale, float *__restrict__ loss,
                                                                   float *__restrict__ dscore) {
    const int lane = threadIdx.x & 63, t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;                                  // (whole waves; nothing below synchronises the workgroup)
    const int nt = nsel[t], K4 = K >> 2;
    const float4 *irow = reinterpret_cast<const float4 *>(sel + (int64_t)t * K);
    const float4 *prow = reinterpret_cast<const float4 *>(mass + (int64_t)t * K);
    float s[NV][4], p[NV][4];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i4 = lane + 64 * u;
        const float4 a = irow[min(i4, K4 - 1)], b = prow[min(i4, K4 - 1)];
        s[u][0] = a.x; s[u][1] = a.y; s[u][2] = a.z; s[u][3] = a.w;
        p[u][0] = b.x; p[u][1] = b.y; p[u][2] = b.z; p[u][3] = b.w;
    }
    float m = -INFINITY;
#pragma unroll
    for (int u = 0; u < NV; ++u)
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (4 * (lane + 64 * u) + c < nt) m = fmaxf(m, s[u][c]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    float z = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u)
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (4 * (lane + 64 * u) + c < nt) z += __expf(s[u][c] - m);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) z += __shfl_xor(z, off, 64);
    const float lse = m + __logf(z);
    float acc = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i4 = lane + 64 * u;
        float g[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            g[c] = 0.f;
            if (4 * i4 + c < nt) {
                const float logq = s[u][c] - lse;
                if (p[u][c] > 0.f) acc += p[u][c] * (__logf(p[u][c]) - logq);
                g[c] = (__expf(logq) - p[u][c]) * grad_scale;
            }
        }
        if (dscore && i4 < K4) reinterpret_cast<float4 *>(dscore + (int64_t)t * K)[i4] = make_float4(g[0], g[1], g[2], g[3]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) loss[t] = nt > 0 ? acc : 0.f;
}

extern "C" hipError_t dsa_launch_indexer_kl(const float *sel, const float *mass, const int32_t *n, int T, int K,
                                            float grad_scale, float *loss, float *dscore, hipStream_t stream) {
    if (T <= 0) return hipSuccess;
    const bool rows16 = K % 4 == 0 && ((reinterpret_cast<uintptr_t>(sel) | reinterpret_cast<uintptr_t>(mass) |
                                        reinterpret_cast<uintptr_t>(dscore)) & 15) == 0;
    const dim3 grid((unsigned)((T + 3) / 4));
#define KL_ROWS(NV) hipLaunchKernelGGL(dsa_indexer_kl_rows_kernel<NV>, grid, dim3(256), 0, stream, sel, mass, n, T, K, grad_scale, loss, dscore)
    if (rows16 && K <= 256) KL_ROWS(1);
    else if (rows16 && K <= 512) KL_ROWS(2);
    else if (rows16 && K <= 1024) KL_ROWS(4);
    else if (rows16 && K <= 2048) KL_ROWS(8);
    else hipLaunchKernelGGL(dsa_indexer_kl_kernel, dim3(T), dim3(256), 0, stream, sel, mass, n, K, grad_scale, loss, dscore);
#undef KL_ROWS
    return hipGetLastError();
}
