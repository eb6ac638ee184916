// Stage D4 (part): pieces of the sparse attention backward that are not tile kernels.
//
//   delta[h,t] = sum_d dO[t,h,d] * O[t,h,d]                                  (dsa_bwd_delta_kernel)
//   p = exp(q.k*scale - lse),  dP = dO.v,  dS = p * (dP - delta)
//   dQ[t]  = scale * sum_{s in sel(t)} dS[t,s] k[s]      query side by gather, one wave per (t, kv head),
//                                                         for the rows where the selection is sparse
//                                                         (dsa_bwd_dq_kernel; dense rows: dsa_tile_dq_kernel)
//   inverted selection: bitmap[t][w] bit b <=> query t selected key column 32w+b of its segment
//                                                         (dsa_bitmap_kernel); the key-side passes
//                                                         dsa_tile_dkv2_kernel / dsa_tile_dkvpc_kernel reduce
//                                                         every key row from it without atomics.
#include "dsa_common.h"

// ------------------------------------------------------------------------------------------------
// delta: 16 lanes per (t,h) row; lane i sums the 8-element chunks i, i+16, ... in one chain, then a butterfly over the 16
// lanes (dsa_tile_dq_kernel reproduces this order when it forms delta itself)
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dsa_bwd_delta_kernel(const bf16_t *__restrict__ dout,
                                                            const bf16_t *__restrict__ out, int T, int Hq, int D,
                                                            float *__restrict__ delta) {
    const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int sub = threadIdx.x & 15;
    float acc = 0.f;
    if (row < (int64_t)T * Hq) {
        for (int c = sub * 8; c < D; c += 128) {
            acc = dot8_chain(load_bf16x8(dout + row * D + c), load_bf16x8(out + row * D + c), acc);
        }
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (sub == 0 && row < (int64_t)T * Hq) {
        const int t = (int)(row / Hq), h = (int)(row % Hq);
        delta[(int64_t)h * T + t] = acc;
    }
}

// ------------------------------------------------------------------------------------------------
// query side: dQ.  Same mapping and operand layouts as the forward kernel; K rows are needed twice
// (row-wise as the A operand of S^T = K Q^T, transposed as the A operand of dQ^T = K^T dS^T), so they
// go HBM -> registers (A layout) -> LDS copy for the transposed 2-byte reads.  V rows are only needed
// row-wise (dP^T = V dO^T) and never touch LDS.
// ------------------------------------------------------------------------------------------------
template <int D, bool HAS_IDX>
__global__ __launch_bounds__(64) void dsa_bwd_dq_kernel(
    const bf16_t *__restrict__ dout, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, const float *__restrict__ lse, const float *__restrict__ delta,
    const int32_t *__restrict__ idx, const int32_t *__restrict__ nsel, const int32_t *__restrict__ cu, int N, int T,
    int Hq, int Hkv, int K, float scale, int pos_min, bf16_t *__restrict__ dq) {
    constexpr int KS = D / 32, DT = D / 16, ROW_B = D * 2 + 8;
    __shared__ __attribute__((aligned(16))) unsigned char klds[32 * ROW_B];

    const int lane = threadIdx.x, g = lane >> 4, m = lane & 15;
    const int kvh = blockIdx.x % Hkv, t = blockIdx.x / Hkv;
    const int G = Hq / Hkv;
    const int s0 = cu[find_segment(cu, N, t)];
    if (t - s0 < pos_min) return;                     // rows before the split belong to the tile kernel
    // the count is held to [0, K] and every row id to the batch: a bad list cannot reach outside the tensors
    const int nt = HAS_IDX ? min(nsel[t], K) : (t - s0 + 1);
    const int32_t *irow = HAS_IDX ? idx + (int64_t)t * K : nullptr;
    if (nt <= 0) {                                    // nothing selected: dQ = 0
        if (m < Hq / Hkv) {
            bf16_t *op = dq + ((int64_t)t * Hq + kvh * (Hq / Hkv) + m) * D + 4 * g;
#pragma unroll
            for (int dt = 0; dt < D / 16; ++dt) *reinterpret_cast<u32x2 *>(op + dt * 16) = u32x2{0u, 0u};
        }
        return;
    }
    auto key_of = [&](int j) -> int {
        j = min(j, nt - 1);
        return HAS_IDX ? min(max(irow[j], 0), T - 1) : s0 + j;
    };
    const float scale_log2 = scale * LOG2E_F;
    const int hq = kvh * G + min(m, G - 1);
    bf16x8 qB[KS], doB[KS];
    {
        const int64_t off = ((int64_t)t * Hq + hq) * D + g * (D / 4);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qB[ks] = (m < G) ? load_bf16x8(q + off + ks * 8) : zero_bf16x8();
            doB[ks] = (m < G) ? load_bf16x8(dout + off + ks * 8) : zero_bf16x8();
        }
    }
    const float lse2 = lse[(int64_t)hq * T + t] * LOG2E_F;
    const float dlt = delta[(int64_t)hq * T + t];

    bf16x8 ka[KS], kb[KS], va[KS], vb[KS];
    auto issue_loads = [&](int myidx) {
        const int ra = __shfl(myidx, m, 64), rb = __shfl(myidx, 16 + m, 64);
        const int64_t oa = ((int64_t)ra * Hkv + kvh) * D + g * (D / 4);
        const int64_t ob = ((int64_t)rb * Hkv + kvh) * D + g * (D / 4);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            ka[ks] = load_bf16x8(k + oa + ks * 8);
            kb[ks] = load_bf16x8(k + ob + ks * 8);
            va[ks] = load_bf16x8(v + oa + ks * 8);
            vb[ks] = load_bf16x8(v + ob + ks * 8);
        }
    };
    f32x4 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int ntiles = (nt + 31) >> 5;
    int idx_next = key_of(lane & 31);
    issue_loads(idx_next);
    idx_next = key_of(32 + (lane & 31));
    for (int it = 0; it < ntiles; ++it) {
        const int j0 = it << 5;
        // K rows -> LDS copy (row m / 16+m, this lane's D/4 slice)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const u32x4 wa = __builtin_bit_cast(u32x4, ka[ks]), wb = __builtin_bit_cast(u32x4, kb[ks]);
            u32x2 *da = reinterpret_cast<u32x2 *>(klds + m * ROW_B + (g * (D / 4) + ks * 8) * 2);
            u32x2 *db = reinterpret_cast<u32x2 *>(klds + (16 + m) * ROW_B + (g * (D / 4) + ks * 8) * 2);
            da[0] = u32x2{wa[0], wa[1]}; da[1] = u32x2{wa[2], wa[3]};
            db[0] = u32x2{wb[0], wb[1]}; db[1] = u32x2{wb[2], wb[3]};
        }
        __syncthreads();
        f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = sa, pa = sa, pb = sa;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            sa = mfma16(ka[ks], qB[ks], sa);
            sb = mfma16(kb[ks], qB[ks], sb);
            pa = mfma16(va[ks], doB[ks], pa);
            pb = mfma16(vb[ks], doB[ks], pb);
        }
        if (it + 1 < ntiles) {
            issue_loads(idx_next);
            idx_next = key_of(j0 + 64 + (lane & 31));
        }
        float ds[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int jpos = j0 + ((e < 4) ? (4 * g + e) : (16 + 4 * g + e - 4));
            const float s = (e < 4) ? sa[e] : sb[e - 4];
            const float dp = (e < 4) ? pa[e] : pb[e - 4];
            const float p = (jpos < nt) ? exp2f(s * scale_log2 - lse2) : 0.f;
            ds[e] = p * (dp - dlt);
        }
        u32x4 dw = {pack2bf(ds[0], ds[1]), pack2bf(ds[2], ds[3]), pack2bf(ds[4], ds[5]), pack2bf(ds[6], ds[7])};
        const bf16x8 dsB = __builtin_bit_cast(bf16x8, dw);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            uint32_t w4[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const int e_lo = 2 * e2, e_hi = 2 * e2 + 1;
                const int r_lo = (e_lo < 4) ? (4 * g + e_lo) : (16 + 4 * g + e_lo - 4);
                const int r_hi = (e_hi < 4) ? (4 * g + e_hi) : (16 + 4 * g + e_hi - 4);
                const uint32_t lo = *reinterpret_cast<const uint16_t *>(klds + r_lo * ROW_B + (dt * 16 + m) * 2);
                const uint32_t hi = *reinterpret_cast<const uint16_t *>(klds + r_hi * ROW_B + (dt * 16 + m) * 2);
                w4[e2] = lo | (hi << 16);
            }
            const bf16x8 aK = __builtin_bit_cast(bf16x8, (u32x4{w4[0], w4[1], w4[2], w4[3]}));
            acc[dt] = mfma16(aK, dsB, acc[dt]);
        }
        __syncthreads();
    }
    if (m < G) {
        bf16_t *op = dq + ((int64_t)t * Hq + kvh * G + m) * D + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            u32x2 w2 = {pack2bf(acc[dt][0] * scale, acc[dt][1] * scale), pack2bf(acc[dt][2] * scale, acc[dt][3] * scale)};
            *reinterpret_cast<u32x2 *>(op + dt * 16) = w2;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// inverted selection: bitmap[t][w] bit b  <=>  key column 32*w+b (relative to the segment start)
// is selected by query t.  One workgroup per query row builds the row in LDS and writes it once.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dsa_bitmap_kernel(const int32_t *__restrict__ idx,
                                                             const int32_t *__restrict__ nsel,
                                                             const int32_t *__restrict__ cu, int N, int K, int ldw,
                                                             uint32_t *__restrict__ bitmap) {
    extern __shared__ uint32_t words[];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int s0 = cu[find_segment(cu, N, t)];
    for (int i = tid; i < ldw; i += 256) words[i] = 0u;
    __syncthreads();
    // entries outside the row's ldw words (a list that names keys of another segment, or a max_seqlen below the
    // longest segment) are dropped, the count is held to K: a caller's mistake cannot write outside the row
    const int nt = min(max(nsel[t], 0), K);
    const unsigned ncols = (unsigned)ldw * 32u;
    const int32_t *irow = idx + (int64_t)t * K;
    // 16-byte loads, all of a thread's in flight (one load per loop iteration would pay the memory latency nt/256 times)
    const int n4 = (reinterpret_cast<uintptr_t>(irow) & 15) ? 0 : nt >> 2;
    const int4 *irow4 = reinterpret_cast<const int4 *>(irow);
    for (int base = 0; base < n4; base += 4 * 256) {
        int4 c4[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) c4[u] = irow4[min(base + u * 256 + tid, n4 - 1)];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (base + u * 256 + tid < n4) {
                const int cs[4] = {c4[u].x - s0, c4[u].y - s0, c4[u].z - s0, c4[u].w - s0};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if ((unsigned)cs[e] < ncols) atomicOr(&words[cs[e] >> 5], 1u << (cs[e] & 31));
            }
    }
    for (int j = (n4 << 2) + tid; j < nt; j += 256) {
        const int c = irow[j] - s0;
        if ((unsigned)c < ncols) atomicOr(&words[c >> 5], 1u << (c & 31));
    }
    __syncthreads();
    uint32_t *orow = bitmap + (int64_t)t * ldw;
    for (int i = tid; i < ldw; i += 256) orow[i] = words[i];
}

// ------------------------------------------------------------------------------------------------
// host-side launchers
// ------------------------------------------------------------------------------------------------
extern "C" hipError_t dsa_launch_delta(const void *dout, const void *out, int T, int Hq, int D, float *delta,
                                       hipStream_t stream) {
    const int64_t rows = (int64_t)T * Hq;
    if (rows == 0) return hipSuccess;
    hipLaunchKernelGGL(dsa_bwd_delta_kernel, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream,
                       (const bf16_t *)dout, (const bf16_t *)out, T, Hq, D, delta);
    return hipGetLastError();
}

extern "C" hipError_t dsa_launch_bitmap(const int32_t *idx, const int32_t *n, const int32_t *cu, int N, int T, int K,
                                        int ldw, uint32_t *bitmap, hipStream_t stream) {
    if (T == 0) return hipSuccess;
    hipLaunchKernelGGL(dsa_bitmap_kernel, dim3(T), dim3(256), (size_t)ldw * 4, stream, idx, n, cu, N, K, ldw, bitmap);
    return hipGetLastError();
}

template <int D>
static hipError_t launch_dq(const void *dout, const void *q, const void *k, const void *v, const float *lse,
                            const float *delta, const int32_t *idx, const int32_t *n, const int32_t *cu, int N, int T,
                            int Hq, int Hkv, int K, float scale, int pos_min, void *dq, hipStream_t stream) {
    const dim3 gq((unsigned)((int64_t)T * Hkv));
    if (idx)
        hipLaunchKernelGGL((dsa_bwd_dq_kernel<D, true>), gq, dim3(64), 0, stream, (const bf16_t *)dout,
                           (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, idx, n, cu, N, T, Hq,
                           Hkv, K, scale, pos_min, (bf16_t *)dq);
    else
        hipLaunchKernelGGL((dsa_bwd_dq_kernel<D, false>), gq, dim3(64), 0, stream, (const bf16_t *)dout,
                           (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, idx, n, cu, N, T, Hq,
                           Hkv, K, scale, pos_min, (bf16_t *)dq);
    return hipGetLastError();
}

extern "C" hipError_t dsa_launch_gather_dq(const void *dout, const void *q, const void *k, const void *v,
                                           const float *lse, const float *delta, const int32_t *idx, const int32_t *n,
                                           const int32_t *cu, int N, int T, int Hq, int Hkv, int D, int K, float scale,
                                           int pos_min, void *dq, hipStream_t stream) {
    if (T == 0) return hipSuccess;
    switch (D) {
        case 64: return launch_dq<64>(dout, q, k, v, lse, delta, idx, n, cu, N, T, Hq, Hkv, K, scale, pos_min, dq, stream);
        case 128: return launch_dq<128>(dout, q, k, v, lse, delta, idx, n, cu, N, T, Hq, Hkv, K, scale, pos_min, dq, stream);
        case 256: return launch_dq<256>(dout, q, k, v, lse, delta, idx, n, cu, N, T, Hq, Hkv, K, scale, pos_min, dq, stream);
        default: return hipErrorInvalidValue;
    }
}
