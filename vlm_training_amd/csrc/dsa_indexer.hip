// Stage D1: lightning-indexer scores on bf16 MFMA.
//
//   score[t,s] = scale * sum_j w[t,j] * relu( q_idx[t,j,:] . k_idx[s,:] ),   s in [seg_start(t), t]
//
// GEMM view: rows = (query, indexer head), columns = keys, contraction = Di.  One wave owns one query:
// its Hi x Di index-query block stays in registers as the A operand of v_mfma_f32_32x32x16_bf16
// (32 heads per tile), key rows stream through LDS in 64-key tiles shared by the four waves of the
// workgroup (double buffered, one barrier per tile).  The epilogue applies ReLU and the per-head
// weight to the 32x32 fp32 tile in registers and reduces over heads (in-lane over 16 rows, then one
// cross-lane add), so only one fp32 per (query,key) pair reaches HBM.  Key tiles outside the query's
// own segment or above its diagonal are skipped per wave; queries whose causal window is not longer
// than top-k are skipped altogether.
#include "dsa_common.h"

__device__ __forceinline__ f32x16 zero_acc() {
    f32x16 z;
#pragma unroll
    for (int v = 0; v < 16; ++v) z[v] = 0.f;
    return z;
}

#define IDX_WAVES 4
#define IDX_BK 64

template <int HT, int DI>
__global__ __launch_bounds__(IDX_WAVES * 64, 2) void dsa_indexer_scores_kernel(
    const bf16_t *__restrict__ q_idx, const bf16_t *__restrict__ k_idx, const bf16_t *__restrict__ w_idx,
    const int32_t *__restrict__ cu, int N, int T, int Hi, float scale, int row_begin, int row_end, int skip_dense_k,
    float *__restrict__ scores, int64_t ld) {
    constexpr int KS = DI / 16;                 // MFMA k-steps
    constexpr int ROW_B = DI * 2 + 16;          // padded LDS row (bytes): conflict-free 16-byte reads
    constexpr int CHUNKS = IDX_BK * DI / 8;     // 16-byte chunks per key tile
    constexpr int LOADS = CHUNKS / (IDX_WAVES * 64);
    static_assert(CHUNKS % (IDX_WAVES * 64) == 0, "tile must split evenly");
    __shared__ __attribute__((aligned(16))) unsigned char lds[2][IDX_BK * ROW_B];
    __shared__ int range_lo[IDX_WAVES], range_hi[IDX_WAVES];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int t = row_begin + blockIdx.x * IDX_WAVES + wv;
    bool active = t < row_end;
    int s0 = 0;
    if (active) {
        s0 = cu[find_segment(cu, N, t)];
        if (t - s0 + 1 <= skip_dense_k) active = false;
    }
    if (lane == 0) { range_lo[wv] = active ? s0 : 0x7fffffff; range_hi[wv] = active ? t : -1; }
    __syncthreads();
    int lo = range_lo[0], hi = range_hi[0];
#pragma unroll
    for (int i = 1; i < IDX_WAVES; ++i) { lo = min(lo, range_lo[i]); hi = max(hi, range_hi[i]); }
    if (hi < 0) return;                          // uniform: nothing to do in this workgroup

    // A operand: this wave's query, heads ht*32 + lane%32, k = ks*16 + 8*(lane/32) + e
    bf16x8 a[HT][KS];
    float wreg[HT][16];
    const int tq = active ? t : 0;
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
        const int head = ht * 32 + (lane & 31);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            a[ht][ks] = (active && head < Hi)
                            ? load_bf16x8(q_idx + ((int64_t)tq * Hi + head) * DI + ks * 16 + (lane >> 5) * 8)
                            : zero_bf16x8();
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int hrow = ht * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
            wreg[ht][v] = (active && hrow < Hi) ? (float)w_idx[(int64_t)tq * Hi + hrow] : 0.f;
        }
    }

    const int kt0 = lo & ~(IDX_BK - 1);
    const int ntiles = (hi - kt0) / IDX_BK + 1;
    u32x4 stage[LOADS];
    auto load_tile = [&](int kt) {
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int c = r * (IDX_WAVES * 64) + tid;
            const int row = c / (DI / 8), col = c % (DI / 8);
            const int krow = min(kt + row, T - 1);           // rows past the batch are never consumed
            stage[r] = *reinterpret_cast<const u32x4 *>(k_idx + (int64_t)krow * DI + col * 8);
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int c = r * (IDX_WAVES * 64) + tid;
            const int row = c / (DI / 8), col = c % (DI / 8);
            *reinterpret_cast<u32x4 *>(&lds[buf][row * ROW_B + col * 16]) = stage[r];
        }
    };
    load_tile(kt0);
    store_tile(0);
    __syncthreads();
    float *orow = scores + (int64_t)(tq - row_begin) * ld;
    for (int it = 0; it < ntiles; ++it) {
        const int kt = kt0 + it * IDX_BK;
        if (it + 1 < ntiles) load_tile(kt + IDX_BK);
        const unsigned char *buf = lds[it & 1];
        if (active) {
            // key operands of sub-tile `sub` (32 keys): all KS reads issued together
            auto read_b = [&](int sub, bf16x8 (&b)[KS]) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    b[ks] = *reinterpret_cast<const bf16x8 *>(buf + (sub * 32 + (lane & 31)) * ROW_B + (ks * 16 + (lane >> 5) * 8) * 2);
            };
            auto gemm = [&](const bf16x8 (&b)[KS], f32x16 (&acc)[HT]) {
#pragma unroll
                for (int ht = 0; ht < HT; ++ht) acc[ht] = zero_acc();
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int ht = 0; ht < HT; ++ht) acc[ht] = mfma32(a[ht][ks], b[ks], acc[ht]);
            };
            // ReLU (one integer max on the bit pattern: negative floats are negative integers; fmaxf would
            // cost a second instruction to quiet NaNs), head weights, sum over heads, store
            auto epilogue = [&](int kb, const f32x16 (&acc)[HT]) {
                float sum = 0.f;
#pragma unroll
                for (int ht = 0; ht < HT; ++ht)
#pragma unroll
                    for (int v = 0; v < 16; ++v) sum += wreg[ht][v] * __int_as_float(max(__float_as_int(acc[ht][v]), 0));
                sum = half_sum_f(sum);
                const int s = kb + (lane & 31);
                if (lane < 32 && s >= s0 && s <= t && s - s0 < ld) orow[s - s0] = sum * scale;   // ld bounds the row whatever the caller's max_seqlen
            };
            const bool on0 = !(kt > t || kt + 31 < s0), on1 = !(kt + 32 > t || kt + 63 < s0);   // wave-uniform
            if (on0 && on1) {
                // both halves of the tile: the second GEMM is issued between the first half's epilogue
                bf16x8 b0[KS], b1[KS];
                f32x16 acc0[HT], acc1[HT];
                read_b(0, b0);
                read_b(1, b1);
                gemm(b0, acc0);
                gemm(b1, acc1);
                epilogue(kt, acc0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * KS, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, KS * HT, 0);
#pragma unroll
                for (int i = 0; i < KS * HT; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, (32 * HT * 2 + KS * HT - 1) / (KS * HT), 0);
                }
                epilogue(kt + 32, acc1);
            } else if (on0 || on1) {
                const int sub = on0 ? 0 : 1;
                bf16x8 b[KS];
                f32x16 acc[HT];
                read_b(sub, b);
                gemm(b, acc);
                __builtin_amdgcn_sched_group_barrier(0x100, KS, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, KS * HT, 0);
                epilogue(kt + 32 * sub, acc);
            }
        }
        if (it + 1 < ntiles) store_tile((it + 1) & 1);
        __syncthreads();
    }
}

template <int HT, int DI>
static hipError_t launch_indexer(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu, int N,
                                 int T, int Hi, float scale, int row_begin, int row_end, int skip_dense_k,
                                 float *scores, int64_t ld, hipStream_t stream) {
    const int rows = row_end - row_begin;
    const int grid = (rows + IDX_WAVES - 1) / IDX_WAVES;
    hipLaunchKernelGGL((dsa_indexer_scores_kernel<HT, DI>), dim3(grid), dim3(IDX_WAVES * 64), 0, stream,
                       (const bf16_t *)q_idx, (const bf16_t *)k_idx, (const bf16_t *)w_idx, cu, N, T, Hi, scale,
                       row_begin, row_end, skip_dense_k, scores, ld);
    return hipGetLastError();
}

// returns hipErrorInvalidValue for geometries the kernel does not cover
extern "C" hipError_t dsa_launch_indexer(const void *q_idx, const void *k_idx, const void *w_idx, const int32_t *cu,
                                         int N, int T, int Hi, int Di, float scale, int row_begin, int row_end,
                                         int skip_dense_k, float *scores, int64_t ld, hipStream_t stream) {
    if (row_end <= row_begin) return hipSuccess;
    const int HT = (Hi + 31) / 32;
#define IDX_CASE(ht, di) \
    if (HT == ht && Di == di) \
        return launch_indexer<ht, di>(q_idx, k_idx, w_idx, cu, N, T, Hi, scale, row_begin, row_end, skip_dense_k, scores, ld, stream);
    IDX_CASE(1, 32) IDX_CASE(1, 64) IDX_CASE(1, 128)
    IDX_CASE(2, 32) IDX_CASE(2, 64) IDX_CASE(2, 128)
#undef IDX_CASE
    return hipErrorInvalidValue;
}
