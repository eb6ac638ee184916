// Stage D4: sparse attention backward, deterministic and atomics-free.
//
//   delta[h,t] = sum_d dO[t,h,d] * O[t,h,d]                                  (dsa_bwd_delta_kernel)
//   p = exp(q.k*scale - lse),  dP = dO.v,  dS = p * (dP - delta)
//   dQ[t]  = scale * sum_{s in sel(t)} dS[t,s] k[s]      query side: same gather as the forward,
//                                                         one wave per (t, kv head)  (dsa_bwd_dq_kernel)
//   dV[s]  = sum_{t: s in sel(t)} p[t,s]^T dO[t]          key side: the selection lists are inverted
//   dK[s]  = scale * sum_{t: s in sel(t)} dS[t,s]^T q[t]  into a bitmap keyed by (query, key column)
//                                                         (dsa_bwd_bitmap_kernel) and every 64-key tile
//                                                         reduces its own contributors in query order
//                                                         (dsa_bwd_dkv_kernel): no atomics, fixed order.
#include "dsa_common.h"

// ------------------------------------------------------------------------------------------------
// delta: 16 lanes per (t,h) row
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dsa_bwd_delta_kernel(const bf16_t *__restrict__ dout,
                                                            const bf16_t *__restrict__ out, int T, int Hq, int D,
                                                            float *__restrict__ delta) {
    const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int sub = threadIdx.x & 15;
    float acc = 0.f;
    if (row < (int64_t)T * Hq) {
        for (int c = sub * 8; c < D; c += 128) {
            const bf16x8 a = load_bf16x8(dout + row * D + c), b = load_bf16x8(out + row * D + c);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc += (float)a[e] * (float)b[e];
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
    int Hq, int Hkv, int K, float scale, bf16_t *__restrict__ dq) {
    constexpr int KS = D / 32, DT = D / 16, ROW_B = D * 2 + 8;
    __shared__ __attribute__((aligned(16))) unsigned char klds[32 * ROW_B];

    const int lane = threadIdx.x, g = lane >> 4, m = lane & 15;
    const int kvh = blockIdx.x % Hkv, t = blockIdx.x / Hkv;
    const int G = Hq / Hkv;
    const int s0 = cu[find_segment(cu, N, t)];
    const int nt = HAS_IDX ? nsel[t] : (t - s0 + 1);
    const int32_t *irow = HAS_IDX ? idx + (int64_t)t * K : nullptr;
    auto key_of = [&](int j) -> int {
        j = min(j, nt - 1);
        return HAS_IDX ? irow[j] : s0 + j;
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
__global__ __launch_bounds__(256) void dsa_bwd_bitmap_kernel(const int32_t *__restrict__ idx,
                                                             const int32_t *__restrict__ nsel,
                                                             const int32_t *__restrict__ cu, int N, int K, int ldw,
                                                             uint32_t *__restrict__ bitmap) {
    extern __shared__ uint32_t words[];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int s0 = cu[find_segment(cu, N, t)];
    for (int i = tid; i < ldw; i += 256) words[i] = 0u;
    __syncthreads();
    const int nt = nsel[t];
    const int32_t *irow = idx + (int64_t)t * K;
    for (int j = tid; j < nt; j += 256) {
        const int c = irow[j] - s0;
        atomicOr(&words[c >> 5], 1u << (c & 31));
    }
    __syncthreads();
    uint32_t *orow = bitmap + (int64_t)t * ldw;
    for (int i = tid; i < ldw; i += 256) orow[i] = words[i];
}

// ------------------------------------------------------------------------------------------------
// key side: dK, dV.  Workgroup = 4 waves = one tile of 64 consecutive keys of one segment and one
// kv head; wave w keeps its 16 keys' K and V rows in registers as MFMA B operands and accumulates
// dK^T / dV^T (fp32) for them.  The workgroup walks the queries t >= tile start of the segment in
// blocks of QB queries; their q / dO rows (G heads each) are staged in LDS once per block and read by
// all four waves in both layouts.  Rows of the MFMA M dimension are (query, head) pairs.
// ------------------------------------------------------------------------------------------------

template <int D, bool HAS_IDX>
__global__ __launch_bounds__(256) void dsa_bwd_dkv_kernel(
    const bf16_t *__restrict__ dout, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, const float *__restrict__ lse, const float *__restrict__ delta,
    const uint32_t *__restrict__ bitmap, int ldw, const int32_t *__restrict__ cu, int N, int T, int Hq, int Hkv,
    int Gp, int gshift, float scale, bf16_t *__restrict__ dk, bf16_t *__restrict__ dv) {
    constexpr int KS = D / 32, DT = D / 16, ROW_B = D * 2 + 8;
    constexpr int DKV_ROWS = (D > 128) ? 32 : 64;    // (query, head) rows per block (LDS budget)
    constexpr int CPR = D / 8;                       // 16-byte chunks per row
    constexpr int LOADS = DKV_ROWS * CPR / 256;      // chunks per thread per operand per block
    __shared__ __attribute__((aligned(16))) unsigned char qlds[DKV_ROWS * ROW_B];
    __shared__ __attribute__((aligned(16))) unsigned char dolds[DKV_ROWS * ROW_B];
    __shared__ float lse_s[DKV_ROWS], dlt_s[DKV_ROWS];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, g = lane >> 4, m = lane & 15;
    const int G = Hq / Hkv;
    const int QB = DKV_ROWS >> gshift;               // queries per block (Gp = 1 << gshift rows each)
    const int kvh = blockIdx.x % Hkv;
    // tile slot -> (segment, 64-key tile): slots are handed out segment by segment
    int slot = blockIdx.x / Hkv, seg = 0, s0 = 0, L = 0;
    for (; seg < N; ++seg) {
        s0 = cu[seg];
        L = cu[seg + 1] - s0;
        const int nt = (L + 63) >> 6;
        if (slot < nt) break;
        slot -= nt;
    }
    if (seg == N) return;                            // spare slot (uniform)
    const int c0 = slot * 64;                        // first key column of the tile
    const int kc = c0 + wv * 16;                     // this wave's first key column
    const int mykey = kc + m;                        // column of MFMA column m
    const bool key_ok = mykey < L;
    const int64_t krow = (int64_t)(s0 + min(mykey, L - 1)) * Hkv + kvh;

    bf16x8 kB[KS], vB[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        kB[ks] = load_bf16x8(k + krow * D + g * (D / 4) + ks * 8);
        vB[ks] = load_bf16x8(v + krow * D + g * (D / 4) + ks * 8);
    }
    f32x4 dkacc[DT], dvacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) { dkacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f}; dvacc[dt] = dkacc[dt]; }

    const float scale_log2 = scale * LOG2E_F;
    u32x4 qst[LOADS], dost[LOADS];
    float lse_st = 0.f, dlt_st = 0.f;
    // block b covers query columns [c0 + b*QB, c0 + (b+1)*QB); row r of the block = (query r>>gshift, head r&(Gp-1))
    auto load_block = [&](int qc0) {
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int c = r * 256 + tid;
            const int row = c / CPR, col = c % CPR;
            const int qc = min(qc0 + (row >> gshift), L - 1);
            const int h = min(row & (Gp - 1), G - 1);
            const int64_t off = ((int64_t)(s0 + qc) * Hq + kvh * G + h) * D + col * 8;
            qst[r] = *reinterpret_cast<const u32x4 *>(q + off);
            dost[r] = *reinterpret_cast<const u32x4 *>(dout + off);
        }
        if (tid < DKV_ROWS) {
            const int qc = min(qc0 + (tid >> gshift), L - 1);
            const int h = min(tid & (Gp - 1), G - 1);
            lse_st = lse[(int64_t)(kvh * G + h) * T + s0 + qc] * LOG2E_F;
            dlt_st = delta[(int64_t)(kvh * G + h) * T + s0 + qc];
        }
    };
    auto store_block = [&]() {
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int c = r * 256 + tid;
            const int row = c / CPR, col = c % CPR;
            u32x2 *dq_ = reinterpret_cast<u32x2 *>(qlds + row * ROW_B + col * 16);
            u32x2 *dd_ = reinterpret_cast<u32x2 *>(dolds + row * ROW_B + col * 16);
            dq_[0] = u32x2{qst[r][0], qst[r][1]}; dq_[1] = u32x2{qst[r][2], qst[r][3]};
            dd_[0] = u32x2{dost[r][0], dost[r][1]}; dd_[1] = u32x2{dost[r][2], dost[r][3]};
        }
        if (tid < DKV_ROWS) { lse_s[tid] = lse_st; dlt_s[tid] = dlt_st; }
    };

    const int nblocks = (L - c0 + QB - 1) / QB;      // queries c0 .. L-1
    load_block(c0);
    for (int b = 0; b < nblocks; ++b) {
        const int qc0 = c0 + b * QB;
        __syncthreads();                              // previous block fully consumed
        store_block();
        __syncthreads();
        if (b + 1 < nblocks) load_block(qc0 + QB);
        // two 16-row sub-tiles per step (32 rows = one K=32 MFMA contraction for dK/dV)
#pragma unroll
        for (int st = 0; st < DKV_ROWS / 32; ++st) {
            const int r0 = st * 32;
            // causal skip: all queries of this step lie before the wave's first key
            if (qc0 + ((r0 + 31) >> gshift) < kc) continue;
            f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = sa, pa = sa, pb = sa;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int cb = (g * (D / 4) + ks * 8) * 2;
                const u32x2 *qa_ = reinterpret_cast<const u32x2 *>(qlds + (r0 + m) * ROW_B + cb);
                const u32x2 *qb_ = reinterpret_cast<const u32x2 *>(qlds + (r0 + 16 + m) * ROW_B + cb);
                const u32x2 *da_ = reinterpret_cast<const u32x2 *>(dolds + (r0 + m) * ROW_B + cb);
                const u32x2 *db_ = reinterpret_cast<const u32x2 *>(dolds + (r0 + 16 + m) * ROW_B + cb);
                const bf16x8 qa = __builtin_bit_cast(bf16x8, (u32x4{qa_[0][0], qa_[0][1], qa_[1][0], qa_[1][1]}));
                const bf16x8 qb = __builtin_bit_cast(bf16x8, (u32x4{qb_[0][0], qb_[0][1], qb_[1][0], qb_[1][1]}));
                const bf16x8 da = __builtin_bit_cast(bf16x8, (u32x4{da_[0][0], da_[0][1], da_[1][0], da_[1][1]}));
                const bf16x8 db = __builtin_bit_cast(bf16x8, (u32x4{db_[0][0], db_[0][1], db_[1][0], db_[1][1]}));
                sa = mfma16(qa, kB[ks], sa);     // S[(t,h) row, key col]
                sb = mfma16(qb, kB[ks], sb);
                pa = mfma16(da, vB[ks], pa);     // dP
                pb = mfma16(db, vB[ks], pb);
            }
            // C layout: lane (key m, group g) holds rows 4g+e (sub-tile a) and 16+4g+e (sub-tile b)
            float pv[8], dsv[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int row = r0 + ((e < 4) ? (4 * g + e) : (16 + 4 * g + e - 4));
                const int qc = qc0 + (row >> gshift);
                const int h = row & (Gp - 1);
                bool on = key_ok && qc < L && h < G && mykey <= qc;
                if (HAS_IDX && on) {
                    const uint32_t wbits = bitmap[(int64_t)(s0 + qc) * ldw + (mykey >> 5)];
                    on = (wbits >> (mykey & 31)) & 1u;
                }
                const float s = (e < 4) ? sa[e] : sb[e - 4];
                const float dp = (e < 4) ? pa[e] : pb[e - 4];
                const float p = on ? exp2f(s * scale_log2 - lse_s[row]) : 0.f;
                pv[e] = p;
                dsv[e] = p * (dp - dlt_s[row]);
            }
            const bf16x8 pB = __builtin_bit_cast(
                bf16x8, (u32x4{pack2bf(pv[0], pv[1]), pack2bf(pv[2], pv[3]), pack2bf(pv[4], pv[5]), pack2bf(pv[6], pv[7])}));
            const bf16x8 dsB = __builtin_bit_cast(
                bf16x8, (u32x4{pack2bf(dsv[0], dsv[1]), pack2bf(dsv[2], dsv[3]), pack2bf(dsv[4], dsv[5]), pack2bf(dsv[6], dsv[7])}));
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                uint32_t wq[4], wd[4];
#pragma unroll
                for (int e2 = 0; e2 < 4; ++e2) {
                    const int e_lo = 2 * e2, e_hi = 2 * e2 + 1;
                    const int r_lo = r0 + ((e_lo < 4) ? (4 * g + e_lo) : (16 + 4 * g + e_lo - 4));
                    const int r_hi = r0 + ((e_hi < 4) ? (4 * g + e_hi) : (16 + 4 * g + e_hi - 4));
                    const int cb = (dt * 16 + m) * 2;
                    wq[e2] = (uint32_t)*reinterpret_cast<const uint16_t *>(qlds + r_lo * ROW_B + cb) |
                             ((uint32_t)*reinterpret_cast<const uint16_t *>(qlds + r_hi * ROW_B + cb) << 16);
                    wd[e2] = (uint32_t)*reinterpret_cast<const uint16_t *>(dolds + r_lo * ROW_B + cb) |
                             ((uint32_t)*reinterpret_cast<const uint16_t *>(dolds + r_hi * ROW_B + cb) << 16);
                }
                const bf16x8 aQ = __builtin_bit_cast(bf16x8, (u32x4{wq[0], wq[1], wq[2], wq[3]}));
                const bf16x8 aD = __builtin_bit_cast(bf16x8, (u32x4{wd[0], wd[1], wd[2], wd[3]}));
                dkacc[dt] = mfma16(aQ, dsB, dkacc[dt]);   // dK^T[d, key] += q^T[d,row] dS[row,key]
                dvacc[dt] = mfma16(aD, pB, dvacc[dt]);    // dV^T[d, key] += dO^T[d,row] P[row,key]
            }
        }
    }
    if (key_ok) {
        bf16_t *pk = dk + krow * D + 4 * g, *pv_ = dv + krow * D + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            u32x2 wk = {pack2bf(dkacc[dt][0] * scale, dkacc[dt][1] * scale), pack2bf(dkacc[dt][2] * scale, dkacc[dt][3] * scale)};
            u32x2 wvv = {pack2bf(dvacc[dt][0], dvacc[dt][1]), pack2bf(dvacc[dt][2], dvacc[dt][3])};
            *reinterpret_cast<u32x2 *>(pk + dt * 16) = wk;
            *reinterpret_cast<u32x2 *>(pv_ + dt * 16) = wvv;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// host-side launchers
// ------------------------------------------------------------------------------------------------
template <int D>
static hipError_t launch_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out,
                             const float *lse, const int32_t *idx, const int32_t *n, const int32_t *cu, int N, int T,
                             int Hq, int Hkv, int K, float scale, int max_seqlen, void *dq, void *dk, void *dv,
                             float *delta, uint32_t *bitmap, int ldw, int parts, hipStream_t stream) {
    const int64_t rows = (int64_t)T * Hq;
    if (parts & 1)
        hipLaunchKernelGGL(dsa_bwd_delta_kernel, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream,
                           (const bf16_t *)dout, (const bf16_t *)out, T, Hq, D, delta);
    const dim3 gq((unsigned)((int64_t)T * Hkv));
    const int G = Hq / Hkv;
    int gshift = 0;
    while ((1 << gshift) < G) ++gshift;
    const int Gp = 1 << gshift;
    const dim3 gk((unsigned)(((int64_t)T / 64 + N + 1) * Hkv));
    if (idx) {
        if (parts & 2)
            hipLaunchKernelGGL(dsa_bwd_bitmap_kernel, dim3(T), dim3(256), (size_t)ldw * 4, stream, idx, n, cu, N, K,
                               ldw, bitmap);
        if (parts & 4)
            hipLaunchKernelGGL((dsa_bwd_dq_kernel<D, true>), gq, dim3(64), 0, stream, (const bf16_t *)dout,
                               (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, idx, n, cu, N, T,
                               Hq, Hkv, K, scale, (bf16_t *)dq);
        if (parts & 8)
            hipLaunchKernelGGL((dsa_bwd_dkv_kernel<D, true>), gk, dim3(256), 0, stream, (const bf16_t *)dout,
                               (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, bitmap, ldw, cu, N,
                               T, Hq, Hkv, Gp, gshift, scale, (bf16_t *)dk, (bf16_t *)dv);
    } else {
        if (parts & 4)
            hipLaunchKernelGGL((dsa_bwd_dq_kernel<D, false>), gq, dim3(64), 0, stream, (const bf16_t *)dout,
                               (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, idx, n, cu, N, T,
                               Hq, Hkv, K, scale, (bf16_t *)dq);
        if (parts & 8)
            hipLaunchKernelGGL((dsa_bwd_dkv_kernel<D, false>), gk, dim3(256), 0, stream, (const bf16_t *)dout,
                               (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, bitmap, ldw, cu, N,
                               T, Hq, Hkv, Gp, gshift, scale, (bf16_t *)dk, (bf16_t *)dv);
    }
    return hipGetLastError();
}

extern "C" hipError_t dsa_launch_attn_bwd(const void *dout, const void *q, const void *k, const void *v,
                                          const void *out, const float *lse, const int32_t *idx, const int32_t *n,
                                          const int32_t *cu, int N, int T, int Hq, int Hkv, int D, int K, float scale,
                                          int max_seqlen, void *dq, void *dk, void *dv, float *delta,
                                          uint32_t *bitmap, int ldw, int parts, hipStream_t stream) {
    if (T == 0) return hipSuccess;
    switch (D) {
        case 64: return launch_bwd<64>(dout, q, k, v, out, lse, idx, n, cu, N, T, Hq, Hkv, K, scale, max_seqlen, dq, dk, dv, delta, bitmap, ldw, parts, stream);
        case 128: return launch_bwd<128>(dout, q, k, v, out, lse, idx, n, cu, N, T, Hq, Hkv, K, scale, max_seqlen, dq, dk, dv, delta, bitmap, ldw, parts, stream);
        case 256: return launch_bwd<256>(dout, q, k, v, out, lse, idx, n, cu, N, T, Hq, Hkv, K, scale, max_seqlen, dq, dk, dv, delta, bitmap, ldw, parts, stream);
        default: return hipErrorInvalidValue;
    }
}
