// Stage D3: sparse attention forward by gathering the selected K/V rows.
//
// One wave (one 64-thread workgroup) per (query token t, kv head).  The G = Hq/Hkv query heads that
// share the kv head are the N columns (padded to 16) of v_mfma_f32_16x16x32_bf16; a tile is 32
// selected keys.
//   S^T[key,h] = K[key,:] . Q[h,:]      A = gathered K rows, read straight from HBM/L2 into the MFMA
//                                       A layout: lane (key m, group g) owns the contiguous D/4
//                                       elements [g*D/4, (g+1)*D/4) of its row (whole 64-byte
//                                       sectors; the contraction order over D is permuted
//                                       identically on the Q side, which does not change the sum)
//   online softmax in fp32 on the C layout (lane = head, 8 keys per lane), exp2 domain
//   O^T[d,h]  += V^T[d,key] . P^T[key,h] A = V rows staged through LDS (16-byte coalesced global reads,
//                                       padded rows, transposed 2-byte reads), B = P^T taken directly
//                                       from the C layout of S^T (no cross-lane movement)
// Loads of tile i+1 are issued before the softmax/PV work of tile i.  blockIdx -> (t, kv head) keeps
// one kv head per XCD (blockIdx % Hkv == XCD % Hkv when Hkv divides 8 or is a multiple of it), so
// every XCD's L2 only sees its own head's K/V.
#include "dsa_common.h"

template <int D, bool HAS_IDX>
__global__ __launch_bounds__(64) void dsa_attn_fwd_kernel(
    const bf16_t *__restrict__ q, const bf16_t *__restrict__ k, const bf16_t *__restrict__ v,
    const int32_t *__restrict__ idx, const int32_t *__restrict__ nsel, const int32_t *__restrict__ cu, int N, int T,
    int Hq, int Hkv, int K, float scale_log2, int pos_min, bf16_t *__restrict__ out, float *__restrict__ lse) {
    constexpr int KS = D / 32;            // MFMA k-steps of the QK^T contraction
    constexpr int DT = D / 16;            // 16-row tiles of O^T
    constexpr int ROW_B = D * 2 + 8;      // padded LDS row: conflict-free transposed reads
    constexpr int CPR = D / 8;            // 16-byte chunks per row
    constexpr int VLOADS = 32 * CPR / 64; // chunks per lane per 32-key tile
    __shared__ __attribute__((aligned(16))) unsigned char vlds[32 * ROW_B];

    const int lane = threadIdx.x, g = lane >> 4, m = lane & 15;
    const int kvh = blockIdx.x % Hkv, t = blockIdx.x / Hkv;
    const int G = Hq / Hkv;
    const int s0 = cu[find_segment(cu, N, t)];
    if (t - s0 < pos_min) return;                             // rows before the split belong to the tile kernel
    // a caller's own list is trusted for its order only: the count is held to [0, K] and every row id to the batch, so
    // that a bad list gives a wrong result, never an access outside the tensors
    const int nt = HAS_IDX ? min(nsel[t], K) : (t - s0 + 1);
    const int32_t *irow = HAS_IDX ? idx + (int64_t)t * K : nullptr;
    if (nt <= 0) {                                            // nothing selected: zero output, lse = -inf
        if (m < G) {
            bf16_t *op = out + ((int64_t)t * Hq + kvh * G + m) * D + 4 * g;
#pragma unroll
            for (int dt = 0; dt < D / 16; ++dt) *reinterpret_cast<u32x2 *>(op + dt * 16) = u32x2{0u, 0u};
            if (g == 0) lse[(int64_t)(kvh * G + m) * T + t] = -INFINITY;
        }
        return;
    }
    auto key_of = [&](int j) -> int {
        j = min(j, nt - 1);                                   // tail columns re-read a valid row, masked below
        return HAS_IDX ? min(max(irow[j], 0), T - 1) : s0 + j;
    };

    bf16x8 qB[KS];
    {
        const bf16_t *qp = q + ((int64_t)t * Hq + kvh * G + min(m, G - 1)) * D + g * (D / 4);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qB[ks] = (m < G) ? load_bf16x8(qp + ks * 8) : zero_bf16x8();
    }

    bf16x8 ka[KS], kb[KS];
    u32x4 vst[VLOADS];
    auto issue_loads = [&](int myidx) {
        const int ra = __shfl(myidx, m, 64), rb = __shfl(myidx, 16 + m, 64);
        const bf16_t *pa = k + ((int64_t)ra * Hkv + kvh) * D + g * (D / 4);
        const bf16_t *pb = k + ((int64_t)rb * Hkv + kvh) * D + g * (D / 4);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) { ka[ks] = load_bf16x8(pa + ks * 8); kb[ks] = load_bf16x8(pb + ks * 8); }
#pragma unroll
        for (int r = 0; r < VLOADS; ++r) {
            const int c = r * 64 + lane;
            const int row = c / CPR, col = c % CPR;
            const int rv = __shfl(myidx, row, 64);
            vst[r] = *reinterpret_cast<const u32x4 *>(v + ((int64_t)rv * Hkv + kvh) * D + col * 8);
        }
    };

    f32x4 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mrun = -INFINITY, lsum = 0.f;

    const int ntiles = (nt + 31) >> 5;
    int idx_next = key_of(lane & 31);
    issue_loads(idx_next);
    idx_next = key_of(32 + (lane & 31));
    for (int it = 0; it < ntiles; ++it) {
        const int j0 = it << 5;
        // V tile -> LDS (row r of the tile = key j0+r)
#pragma unroll
        for (int r = 0; r < VLOADS; ++r) {
            const int c = r * 64 + lane;
            const int row = c / CPR, col = c % CPR;
            u32x2 *dst = reinterpret_cast<u32x2 *>(vlds + row * ROW_B + col * 16);
            dst[0] = u32x2{vst[r][0], vst[r][1]};
            dst[1] = u32x2{vst[r][2], vst[r][3]};
        }
        __syncthreads();
        f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            sa = mfma16(ka[ks], qB[ks], sa);
            sb = mfma16(kb[ks], qB[ks], sb);
        }
        if (it + 1 < ntiles) {
            issue_loads(idx_next);
            idx_next = key_of(j0 + 64 + (lane & 31));
        }
        // online softmax: this lane holds head m, keys j0+4g+e (e<4) and j0+16+4g+(e-4)
        float s2[8];
        float mloc = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int jpos = j0 + ((e < 4) ? (4 * g + e) : (16 + 4 * g + e - 4));
            const float x = ((e < 4) ? sa[e] : sb[e - 4]) * scale_log2;
            s2[e] = (jpos < nt) ? x : -INFINITY;
            mloc = fmaxf(mloc, s2[e]);
        }
        mloc = fmaxf(mloc, wave_xor_f(mloc, 16));
        mloc = half_max_f(mloc);
        const float mnew = fmaxf(mrun, mloc);             // finite: key j0 is always valid
        const float alpha = exp2f(mrun - mnew);
        float psum = 0.f;
        float p[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) { p[e] = exp2f(s2[e] - mnew); psum += p[e]; }
        lsum = lsum * alpha + psum;
        mrun = mnew;
        u32x4 pw = {pack2bf(p[0], p[1]), pack2bf(p[2], p[3]), pack2bf(p[4], p[5]), pack2bf(p[6], p[7])};
        const bf16x8 pB = __builtin_bit_cast(bf16x8, pw);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            oacc[dt] *= alpha;
            uint32_t w4[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const int e_lo = 2 * e2, e_hi = 2 * e2 + 1;
                const int r_lo = (e_lo < 4) ? (4 * g + e_lo) : (16 + 4 * g + e_lo - 4);
                const int r_hi = (e_hi < 4) ? (4 * g + e_hi) : (16 + 4 * g + e_hi - 4);
                const uint32_t lo = *reinterpret_cast<const uint16_t *>(vlds + r_lo * ROW_B + (dt * 16 + m) * 2);
                const uint32_t hi = *reinterpret_cast<const uint16_t *>(vlds + r_hi * ROW_B + (dt * 16 + m) * 2);
                w4[e2] = lo | (hi << 16);
            }
            const bf16x8 aV = __builtin_bit_cast(bf16x8, (u32x4{w4[0], w4[1], w4[2], w4[3]}));
            oacc[dt] = mfma16(aV, pB, oacc[dt]);
        }
        __syncthreads();
    }
    float l = lsum;
    l += wave_xor_f(l, 16);
    l = half_sum_f(l);
    const float inv = 1.f / l;
    if (m < G) {
        bf16_t *op = out + ((int64_t)t * Hq + kvh * G + m) * D + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            u32x2 w2 = {pack2bf(oacc[dt][0] * inv, oacc[dt][1] * inv), pack2bf(oacc[dt][2] * inv, oacc[dt][3] * inv)};
            *reinterpret_cast<u32x2 *>(op + dt * 16) = w2;
        }
        if (g == 0) lse[(int64_t)(kvh * G + m) * T + t] = (mrun + log2f(l)) * LN2_F;
    }
}

template <int D>
static hipError_t launch_fwd(const void *q, const void *k, const void *v, const int32_t *idx, const int32_t *n,
                             const int32_t *cu, int N, int T, int Hq, int Hkv, int K, float scale, int pos_min,
                             void *out, float *lse, hipStream_t stream) {
    const dim3 grid((unsigned)((int64_t)T * Hkv)), block(64);
    const float sl2 = scale * LOG2E_F;
    if (idx)
        hipLaunchKernelGGL((dsa_attn_fwd_kernel<D, true>), grid, block, 0, stream, (const bf16_t *)q, (const bf16_t *)k,
                           (const bf16_t *)v, idx, n, cu, N, T, Hq, Hkv, K, sl2, pos_min, (bf16_t *)out, lse);
    else
        hipLaunchKernelGGL((dsa_attn_fwd_kernel<D, false>), grid, block, 0, stream, (const bf16_t *)q,
                           (const bf16_t *)k, (const bf16_t *)v, idx, n, cu, N, T, Hq, Hkv, K, sl2, pos_min, (bf16_t *)out, lse);
    return hipGetLastError();
}

extern "C" hipError_t dsa_launch_attn_fwd(const void *q, const void *k, const void *v, const int32_t *idx,
                                          const int32_t *n, const int32_t *cu, int N, int T, int Hq, int Hkv, int D,
                                          int K, float scale, int pos_min, void *out, float *lse, hipStream_t stream) {
    if (T == 0) return hipSuccess;
    switch (D) {
        case 64: return launch_fwd<64>(q, k, v, idx, n, cu, N, T, Hq, Hkv, K, scale, pos_min, out, lse, stream);
        case 128: return launch_fwd<128>(q, k, v, idx, n, cu, N, T, Hq, Hkv, K, scale, pos_min, out, lse, stream);
        case 256: return launch_fwd<256>(q, k, v, idx, n, cu, N, T, Hq, Hkv, K, scale, pos_min, out, lse, stream);
        default: return hipErrorInvalidValue;
    }
}
