// Tile kernels: attention forward / dQ / dK,dV over 32x32 MFMA tiles with the selection applied as a
// bitmap mask.  They do the same arithmetic as the gather kernels but visit every (query block, key
// tile) pair of the causal triangle, so they win wherever the selection is dense: one selected pair
// costs the gather kernels 2*D*e bytes of L2 traffic per kv head, a causal pair costs these kernels
// 4*G*D flop on the matrix cores - on MI355X the tile walk is cheaper down to a few percent density.
//
// Common scheme (wave64, v_mfma_f32_32x32x16_bf16):
//   rows of the problem are (query, head-in-group) pairs, `Gp` (power of two >= G) rows per query;
//   the mask depends on the query only.  Operands that move (K,V tiles for the query-stationary
//   kernels, q,dO blocks for the key-stationary one) are staged once per workgroup in LDS, row-major
//   with an XOR swizzle of the 16-byte chunks, and read either row-wise (16-byte reads, contraction
//   over D) or transposed with ds_read_b64_tr_b16 (contraction over rows/keys) - both conflict-free.
//   The second GEMM of each chain takes its B operand straight from the C layout of the first
//   (the contraction order over the 32 keys/rows of a tile is permuted identically on both operands).
#include "dsa_common.h"
#include <type_traits>

typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }   // v_exp_f32; exp2(-inf) = 0

// ---- LDS tile: 32 rows of D bf16 with a pitch of D*2 + 64 bytes (+ 128 at head_dim 96); chunk = 16 bytes ----
// The LDS of gfx950 has 64 four-byte banks (256 B per clock).  A 16-byte read is served 16 lanes at a
// time and a transposed 8-byte read 32 lanes at a time, so a row-wise operand read (16 consecutive rows,
// same chunk) and a transposed read (4 consecutive rows x 64 B) must each cover all banks once.  The
// 64-byte skew per row separates 4 consecutive rows, the XOR of the chunk's two low bits with row bits
// 2-3 separates rows 4 apart: both read patterns and the row-wise staging writes are conflict-free.
// (The skew needs a pitch of 64 modulo 256 bytes: head_dim 96 pads its rows to the pitch of head_dim 128.)
template <int D> constexpr int tile_pitch() { return D == 96 ? 320 : D * 2 + 64; }
template <int D> constexpr int tile_bytes() { return 32 * tile_pitch<D>(); }
__device__ __forceinline__ int tile_sw(int row) { return (row >> 2) & 3; }
template <int D>
__device__ __forceinline__ int tile_off(int row, int chunk) { return row * tile_pitch<D>() + ((chunk ^ tile_sw(row)) << 4); }

// accumulate in place (kept as a function so that the accumulation sites read alike)
__device__ __forceinline__ void mfma32_acc(f32x16 &c, bf16x8 a, bf16x8 b) { c = mfma32(a, b, c); }
// all-ones if bit `b` of `word` is set, else 0 (v_bfe_i32 when b is a compile-time constant)
__device__ __forceinline__ uint32_t bit_mask(uint32_t word, int b) {
    return (uint32_t)(((int32_t)(word << (31 - b))) >> 31);
}
// x where keep is all-ones, -inf where it is 0 (one v_bfi_b32 / v_bitop3_b32)
__device__ __forceinline__ float keep_or_neginf(float x, uint32_t keep) {
    return __uint_as_float((keep & __float_as_uint(x)) | (~keep & 0xff800000u));
}
// bits j <= d of a 32-key tile (keys at or before the diagonal when d = query column - tile start)
__device__ __forceinline__ uint32_t causal_bits(int d) { return d >= 31 ? 0xffffffffu : (d < 0 ? 0u : ((2u << d) - 1u)); }
// Issue order for a chain of NM MFMAs that each consume RPM LDS reads: keep AHEAD MFMAs' worth of reads
// in flight (the machine scheduler otherwise sinks every read next to its use and the chain runs at
// LDS latency).  Applies to the instructions of the enclosing basic block, in program order.
template <int NM, int AHEAD, int RPM, int FIRST = 0>
__device__ __forceinline__ void sched_reads_ahead() {
    __builtin_amdgcn_sched_group_barrier(0x100, FIRST + AHEAD * RPM, 0);   // FIRST: other reads issued up front
#pragma unroll
    for (int i = 0; i < NM - AHEAD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, RPM, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
}
// Per-lane LDS byte offsets of the two read patterns, computed once per kernel so that every operand
// read in the loops is "tile base + lane offset + immediate" (the swizzle only XORs chunk bits 0-1, so
// k-step / d-tile indices move the address by a lane constant plus a compile-time multiple of 64 B).
//   row-wise A operand of mfma32: lane (i = row j, h) takes elements [16*ks + 8h, +8) of row j
//   transposed A operand: lane l takes column c = 32*dt + (l & 31)... of the 8 rows {R..R+3, R+8..R+11}.
//   ds_read_b64_tr_b16: within 16 lanes, lane s supplies the address of 4 consecutive elements of row
//   R + s/4 at column m0 + 4*(s%4); lane s receives rows R..R+3 of column m0 + s.
typedef __attribute__((address_space(3))) unsigned char lds_u8;
template <int D>
struct LaneOffsets {
    int row[2];      // row-wise operand of row j: k-steps ks with ks % 2 == c
    int tr[4];       // transposed operand: rows 4h + s/4 + {0, 8, 16, 24}
    __device__ __forceinline__ void init(int lane) {
        const int h = lane >> 5, j = lane & 31, s = lane & 15;
        const int swj = tile_sw(j);
#pragma unroll
        for (int c = 0; c < 2; ++c) row[c] = j * tile_pitch<D>() + ((((c ^ (swj >> 1)) << 1) | (h ^ (swj & 1))) << 4);
        const int low = ((lane >> 4) & 1) * 2 + ((s & 3) >> 1), sub = (s & 1) << 3;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int r = 4 * h + (s >> 2) + 8 * v;
            tr[v] = r * tile_pitch<D>() + ((low ^ tile_sw(r)) << 4) + sub;
        }
    }
    // row-wise A operand of k-step ks (elements [16ks + 8h, +8) of row j)
    __device__ __forceinline__ bf16x8 rowop(const unsigned char *tile, int ks) const {
        return *reinterpret_cast<const bf16x8 *>(tile + row[ks & 1] + (ks >> 1) * 64);
    }
    __device__ __forceinline__ static bf16x8 tr_pair(lds_u8 *p0, lds_u8 *p1) {
        const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p0);
        const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)p1);
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        const s16x8 r = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
        return __builtin_bit_cast(bf16x8, r);
    }
    // transposed A operand of d-tile dt over rows {R..R+3, R+8..R+11}, R = 4h (pair 0) or 16 + 4h (pair 1)
    __device__ __forceinline__ bf16x8 trop(const unsigned char *tile, int pair, int dt) const {
        return tr_pair((lds_u8 *)tile + tr[2 * pair] + dt * 64, (lds_u8 *)tile + tr[2 * pair + 1] + dt * 64);
    }
    // same with the lane addresses already formed (p[v] = tile + tr[v]): one immediate per read
    __device__ __forceinline__ static bf16x8 trop_at(lds_u8 *const *p, int pair, int dt, int imm) {
        return tr_pair(p[2 * pair] + dt * 64 + imm, p[2 * pair + 1] + dt * 64 + imm);
    }
};
__device__ __forceinline__ bf16x8 pack8(const float *x) {
    const u32x4 w = {pack2bf(x[0], x[1]), pack2bf(x[2], x[3]), pack2bf(x[4], x[5]), pack2bf(x[6], x[7])};
    return __builtin_bit_cast(bf16x8, w);
}
__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int v = 0; v < 16; ++v) z[v] = 0.f;
    return z;
}

// Write one 32-column d-tile of a C-layout accumulator as bf16 (lane = row j; a lane holds the four
// columns 8*g4 + 4*h + {0..3} of every group g4, so a 16-byte chunk of the row is split over the two
// lanes 32 apart).  The halves of the wave exchange 8-byte pieces - lane (j,0) takes chunk 2m whole,
// lane (j,1) chunk 2m+1 - and every lane stores 16 bytes.  Both lanes of a row must be active.
__device__ __forceinline__ void store_c_tile(bf16_t *row_dt, const f32x16 &acc, float mul, int h) {
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        const uint32_t a0 = pack2bf(acc[8 * m] * mul, acc[8 * m + 1] * mul), a1 = pack2bf(acc[8 * m + 2] * mul, acc[8 * m + 3] * mul);
        const uint32_t b0 = pack2bf(acc[8 * m + 4] * mul, acc[8 * m + 5] * mul), b1 = pack2bf(acc[8 * m + 6] * mul, acc[8 * m + 7] * mul);
        const auto r0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);   // upper lanes of a <-> lower lanes of b
        const auto r1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
        const u32x4 w = {r0[0], r1[0], r0[1], r1[1]};
        *reinterpret_cast<u32x4 *>(row_dt + 8 * (2 * m + h)) = w;
    }
}

// slot -> (segment, block) for blocks of `blk` columns handed out segment by segment; within a segment
// the blocks are numbered from the end when `reverse` (heaviest causal blocks first).  Returns false
// for spare slots.  The segment bounds are fetched 64 segments at a time, one per lane (one memory
// round trip instead of one per segment), and walked with lane reads.
__device__ __forceinline__ bool locate_block(const int32_t *cu, int N, int slot, int blk, bool reverse, int &s0, int &L,
                                             int &b) {
    const int lane = threadIdx.x & 63;
    for (int base = 0; base < N; base += 64) {
        const int seg = min(base + lane, N - 1);
        const int lo = cu[seg], len = cu[seg + 1] - lo;
        const int cnt = min(64, N - base);
        for (int w = 0; w < cnt; ++w) {
            L = __builtin_amdgcn_readlane(len, w);
            const int nb = (L + blk - 1) / blk;
            if (slot < nb) {
                s0 = __builtin_amdgcn_readlane(lo, w);
                b = reverse ? nb - 1 - slot : slot;
                return true;
            }
            slot -= nb;
        }
    }
    return false;
}

// The same hand-out, heaviest block first over the whole batch: slot 0 takes the last block of the longest segment,
// then every block with the next lower index in segment order, and so on - a block's walk grows with its index, so
// long walks start first wherever their segment lies in the batch (with the segment-by-segment order the long
// walks of a late segment start late and the launch ends on them).  For up to 64 segments (their lengths live in
// one wave's lanes); larger batches fall back to the segment-by-segment order.
__device__ __forceinline__ int wave_sum_i(int x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}
__device__ __forceinline__ bool locate_block_heaviest_first(const int32_t *cu, int N, int slot, int blk, int &s0, int &L,
                                                            int &b) {
    if (N > 64) return locate_block(cu, N, slot, blk, true, s0, L, b);
    const int lane = threadIdx.x & 63;
    const int seg = min(lane, N - 1);
    const int lo = cu[seg], len = cu[seg + 1] - lo;
    const int nb = lane < N ? (len + blk - 1) / blk : 0;
    int most = nb;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) most = max(most, __shfl_xor(most, off, 64));
    // blocks with index >= x over all segments
    auto count_ge = [&](int x) { return wave_sum_i(max(nb - x, 0)); };
    if (slot >= count_ge(0)) return false;
    int lo_b = 0, hi_b = most;                           // count_ge(lo_b) > slot >= count_ge(hi_b)
    while (hi_b - lo_b > 1) {
        const int mid = (lo_b + hi_b) >> 1;
        if (count_ge(mid) > slot) lo_b = mid; else hi_b = mid;
    }
    b = lo_b;
    const int rank = slot - count_ge(b + 1);             // among the segments that have a block b, in segment order
    const uint64_t has = __builtin_amdgcn_ballot_w64(nb > b);
    // the rank-th set bit of `has`
    const int below = (int)__popcll(has & ((1ull << lane) - 1ull));
    const uint64_t me = __builtin_amdgcn_ballot_w64(nb > b && below == rank);
    const int w = (int)__builtin_ctzll(me);
    s0 = __builtin_amdgcn_readlane(lo, w);
    L = __builtin_amdgcn_readlane(len, w);
    return true;
}

// Query blocks are handed out heaviest first: over the whole batch for launches of a few rounds of workgroups (they
// would otherwise end on the long walks of a late segment: forward -11 %, dQ -15 % on 8192 tokens in seven
// segments), segment by segment for larger ones, where the blocks of a segment that run side by side share their
// K / V tiles in L2 (the batch-wide order is 2-3 % slower there).
#define DSA_BATCH_ORDER_MAX_BLOCKS (6 * 256)
#define LOCATE_QUERY_BLOCK(cu, N, slot, blk, s0, L, b)                                                           \
    (gridDim.x <= DSA_BATCH_ORDER_MAX_BLOCKS ? locate_block_heaviest_first(cu, N, slot, blk, s0, L, b)          \
                                             : locate_block(cu, N, slot, blk, true, s0, L, b))

// ==================================================================================================
// forward: query-stationary.  Workgroup = 4 waves x 32 rows = 128 rows = 128/Gp queries of one
// segment and one kv head; loops over 32-key tiles of the causal range.
//   S^T[key,row] = K[key,:].Q[row,:]   (A = K tile row-wise from LDS, B = Q^T in registers)
//   online softmax on the C layout (lane = row; one cross-lane step per statistic)
//   O^T[d,row]  += V^T[d,key] P^T[key,row]   (A = V tile transposed from LDS, B = P^T from the C layout)
// K/V tiles are fetched two tiles ahead into registers and one tile ahead into LDS (double buffer),
// so a global load has two tile-times to land; one barrier per tile.
// ==================================================================================================
// Every global load of the pipeline is issued unconditionally (indices past the end are clamped to
// the last tile) and nothing is computed from a loaded value before the matching STORE, so the
// compiler can wait with exact vmcnt counts and a load has two tile-times to land.  The kernel issues
// LOAD(0, 0) itself, before the loads of its stationary rows.
#define TILE_PIPELINE(NT, LOAD, STORE, COMPUTE)                                                     \
    {                                                                                              \
        const int nt_last = (NT) - 1;                                                              \
        STORE(0, 0, 0);                                                                            \
        LOAD(0, min(1, nt_last));                                                                  \
        LOAD(1, min(2, nt_last));                                                                  \
        __syncthreads();                                                                           \
        int it = 0;                                                                                \
        for (; it + 1 < (NT); it += 2) {                                                           \
            /* LDS buffer 0 holds tile it, register set 0 tile it+1, register set 1 tile it+2 */     \
            COMPUTE(it, 0);                                                                        \
            if (NBUF == 1) __syncthreads();                                                        \
            STORE(0, NBUF - 1, it + 1);                                                            \
            LOAD(0, min(it + 3, nt_last));                                                         \
            __syncthreads();                                                                       \
            COMPUTE(it + 1, NBUF - 1);                                                             \
            if (NBUF == 1) __syncthreads();                                                        \
            STORE(1, 0, min(it + 2, nt_last));                                                     \
            LOAD(1, min(it + 4, nt_last));                                                         \
            __syncthreads();                                                                       \
        }                                                                                          \
        if (it < (NT)) COMPUTE(it, 0);                                                             \
    }

template <int D, bool HAS_IDX, int GSHIFT, int NW>
__global__ __launch_bounds__(NW * 64, (D <= 128 && NW == 4) ? 2 : 1) void dsa_tile_fwd_kernel(
    const bf16_t *__restrict__ q, const bf16_t *__restrict__ k, const bf16_t *__restrict__ v,
    const uint32_t *__restrict__ bitmap, int ldw, const int32_t *__restrict__ cu, int N, int T, int Hq, int Hkv,
    float scale_log2, int pos_split, int causal, bf16_t *__restrict__ out, float *__restrict__ lse) {
    constexpr int KS = D / 16, DT = D / 32, CPR = D / 8, TILE_B = tile_bytes<D>();
    constexpr int NBUF = (D > 128) ? 1 : 2;           // double buffering where 64 KiB of static LDS allow it
    constexpr int NT = NW * 64, Gp = 1 << GSHIFT, QBW = (NW * 32) >> GSHIFT;
    constexpr int CH = 32 * CPR, LOADS = (CH + NT - 1) / NT;   // 16-byte chunks per matrix; per thread (head_dim 96: not all threads)
    static_assert(CH % 64 == 0, "whole waves stage or do not");
    __shared__ __attribute__((aligned(16))) unsigned char lds[NBUF][2][TILE_B];   // [buffer][K|V]

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, h = lane >> 5, j = lane & 31;
    LaneOffsets<D> lo;
    lo.init(lane);
    const int G = Hq / Hkv;
    const int kvh = blockIdx.x % Hkv;
    int s0, L, blk;
    if (!LOCATE_QUERY_BLOCK(cu, N, blockIdx.x / Hkv, QBW, s0, L, blk)) return;
    if (HAS_IDX) L = min(L, ldw * 32);                  // a bitmap row has ldw words whatever the caller's max_seqlen
    const int qc0 = blk * QBW;
    if (qc0 >= pos_split || qc0 >= L) return;                       // rows past the split belong to the gather kernel

    const int r = wv * 32 + j;
    const int qcol = qc0 + (r >> GSHIFT), head = r & (Gp - 1);
    const bool row_ok = qcol < L && head < G;
    const int t = s0 + min(qcol, L - 1), hq = kvh * G + min(head, G - 1);
    u32x4 kst[2][LOADS], vst[2][LOADS];
#define FWD_LOAD(SET, TILE)                                                                         \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) if (CH % NT == 0 || i * NT + tid < CH) {     \
        const int c = i * NT + tid;                                                               \
        const int row = c / CPR, ch = c % CPR;                                                     \
        const int64_t off = ((int64_t)(s0 + min((TILE) * 32 + row, L - 1)) * Hkv + kvh) * D + ch * 8; \
        kst[SET][i] = *reinterpret_cast<const u32x4 *>(k + off);                                   \
        vst[SET][i] = *reinterpret_cast<const u32x4 *>(v + off);                                   \
    }
    FWD_LOAD(0, 0)                                      // ahead of the q rows: staging waits for this tile only
    bf16x8 qB[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qB[ks] = row_ok ? load_bf16x8(q + ((int64_t)t * Hq + hq) * D + 16 * ks + 8 * h) : zero_bf16x8();
    const int ntiles = (causal ? min(qc0 + QBW - 1, L - 1) : L - 1) / 32 + 1;
    const int klim = causal ? qcol : L - 1;             // last key column this row may attend (dense mode)
    const uint32_t *wrow = bitmap + (int64_t)t * ldw;

    f32x16 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = zero16();
    float mrun = -INFINITY, lsum = 0.f;
    uint32_t word_next = HAS_IDX ? wrow[0] : 0u;        // unconditional loads; rows that are not live are masked at use

#define FWD_STORE(SET, BUF, TILE)                                                                        \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) if (CH % NT == 0 || i * NT + tid < CH) {     \
        const int c = i * NT + tid;                                                               \
        const int row = c / CPR, ch = c % CPR;                                                     \
        *reinterpret_cast<u32x4 *>(&lds[BUF][0][tile_off<D>(row, ch)]) = kst[SET][i];              \
        *reinterpret_cast<u32x4 *>(&lds[BUF][1][tile_off<D>(row, ch)]) = vst[SET][i];              \
    }
// Online softmax of one tile.  The row maximum is not searched in every tile: P is formed against the running
// reference first, and only when a lane's sum says that some probability may have passed 2^8 - or a live row has not met
// a selected key yet - does the wave look for the tile's maximum, move the reference, rescale the sums and form P
// again: the first tile of a block, then rarely.  In between P stays below 2^8, exact in fp32 and safe in bf16, and
// never underflows as a whole, because the reference is a maximum the row has really met.  (Searching the maximum in
// every tile, 16 more vector instructions per tile, was 4-5 % slower at 32 768 tokens.)
#define FWD_SOFTMAX                                                                                \
        float s2[16], pr[16];                                                                      \
        _Pragma("unroll") for (int vi = 0; vi < 16; ++vi)                                          \
            s2[vi] = keep_or_neginf(sacc[vi], bit_mask(word, 8 * (vi >> 2) + (vi & 3)));           \
        float psum = 0.f;                                                                          \
        {                                                                                          \
            const float mneg = (mrun == -INFINITY) ? 0.f : -mrun;                                  \
            _Pragma("unroll") for (int vi = 0; vi < 16; ++vi) {                                    \
                pr[vi] = fast_exp2(fmaf(s2[vi], scale_log2, mneg));                                \
                psum += pr[vi];                                                                    \
            }                                                                                      \
        }                                                                                          \
        if (__builtin_amdgcn_ballot_w64(row_ok && (mrun == -INFINITY || !(psum <= 256.f)))) {      \
            float mloc = -INFINITY;                                                                \
            _Pragma("unroll") for (int vi = 0; vi < 16; ++vi) mloc = fmaxf(mloc, s2[vi]);          \
            mloc = half_max_f(mloc) * scale_log2;                                                  \
            if (mloc > mrun) {                                                                     \
                const float alpha = fast_exp2(mrun - mloc);   /* mrun = -inf: 0, and the sums are 0 */ \
                lsum *= alpha;                                                                     \
                _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) oacc[dt] *= alpha;               \
                mrun = mloc;                                                                       \
            }                                                                                      \
            const float mneg = (mrun == -INFINITY) ? 0.f : -mrun;                                  \
            psum = 0.f;                                                                            \
            _Pragma("unroll") for (int vi = 0; vi < 16; ++vi) {                                    \
                pr[vi] = fast_exp2(fmaf(s2[vi], scale_log2, mneg));                                \
                psum += pr[vi];                                                                    \
            }                                                                                      \
        }                                                                                          \
        lsum += psum;                                                                              \
        const bf16x8 pB0 = pack8(pr), pB1 = pack8(pr + 8);
#define FWD_COMPUTE(TILE, BUF)                                                                      \
    {                                                                                              \
        const int kc0 = (TILE) * 32;                                                               \
        const unsigned char *kt = lds[BUF][0], *vt = lds[BUF][1];                                  \
        uint32_t word = row_ok ? word_next : 0u;                                                   \
        if (HAS_IDX) word_next = wrow[min((TILE) + 1, ntiles - 1)];                                \
        if (!HAS_IDX) word = row_ok ? causal_bits(klim - kc0) : 0u;                                \
        word >>= 4 * h;                                  /* element vi then sits at bit 8*(vi/4) + vi%4 */ \
        f32x16 sacc = zero16();                                                                    \
        {                                                /* all K operands in flight before the first MFMA */ \
            bf16x8 ka[KS];                                                                         \
            _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) ka[ks] = lo.rowop(kt, ks); \
            _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) sacc = mfma32(ka[ks], qB[ks], sacc); \
            sched_reads_ahead<KS, 4, 1>();                                                         \
        }                                                                                          \
        FWD_SOFTMAX                                                                                \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) {                                        \
            mfma32_acc(oacc[dt], lo.trop(vt, 0, dt), pB0);                          \
            mfma32_acc(oacc[dt], lo.trop(vt, 1, dt), pB1);                     \
        }                                                                                          \
        sched_reads_ahead<2 * DT, 3, 2>();                                                         \
    }
    TILE_PIPELINE(ntiles, FWD_LOAD, FWD_STORE, FWD_COMPUTE)
#undef FWD_LOAD
#undef FWD_STORE
#undef FWD_COMPUTE
#undef FWD_SOFTMAX

    float l = half_sum_f(lsum);
    if (row_ok) {
        const float inv = 1.f / l;
        bf16_t *op = out + ((int64_t)t * Hq + hq) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) store_c_tile(op + dt * 32, oacc[dt], inv, h);
        if (h == 0) lse[(int64_t)hq * T + t] = (mrun + log2f(l)) * LN2_F;
    }
}

// ==================================================================================================
// attention mass: the indexer's training target.  Same walk and S^T = K Q^T as the forward, with the
// saved log-sum-exp instead of the online softmax and no V: P = exp(S*scale - lse) on the selected
// keys, summed over the heads of a query that share the kv head (lanes of one query are adjacent:
// DPP adds), and written to the slot the key has in the query's ascending selection list
// (slot = selected keys of earlier tiles + selected keys below it in the tile's word).  One partial
// (T,K) table per kv head; dsa_mass_reduce_kernel adds them in a fixed order.
// ==================================================================================================
template <int CTRL>
__device__ __forceinline__ float dpp_f(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false));
}
// sum over the aligned group of 2^GSHIFT adjacent lanes, on every lane of the group
template <int GSHIFT>
__device__ __forceinline__ float group_sum(float x) {
    if (GSHIFT >= 1) x += dpp_f<0xB1>(x);               // quad_perm [1,0,3,2]
    if (GSHIFT >= 2) x += dpp_f<0x4E>(x);               // quad_perm [2,3,0,1]
    if (GSHIFT >= 3) x += dpp_f<0x141>(x);              // row_half_mirror: the other quad's total
    if (GSHIFT >= 4) x += dpp_f<0x140>(x);              // row_mirror: the other half row's total
    return x;
}
// The heads of a query meet in one workgroup: a wave's 32 rows are (query, head of one kv group) pairs as in the
// forward, and the workgroup takes its HPG kv heads *inside* each key tile - all their K tiles are staged together,
// all their q rows stay in registers - and adds their probabilities up in registers.  With two or more kv heads the
// workgroup has two sets of four waves on the same queries, each set taking half of the kv heads (two waves per
// SIMD: one's exponentials run beside the other's matrix work; a wave holds up to 128 registers of q rows); the
// second set hands its sums to the first through LDS once per tile.  A slot of the result is therefore written
// once, by one lane, with the finished sum: no table per kv head, nothing read back.  Only a batch with more kv
// heads than a workgroup holds is cut into groups with one table each.
template <int D> constexpr int mass_heads_max() { return 1024 / D; }      // 16 / 8 / 4 kv heads at head_dim 64 / 128 / 256
template <int HPG> constexpr int mass_sets() { return HPG >= 2 ? 2 : 1; }
template <int D, int HPG> constexpr size_t mass_lds_bytes() {
    return (size_t)HPG * tile_bytes<D>() + (mass_sets<HPG>() == 2 ? 4 * 64 * 16 * sizeof(float) : 0);
}
template <int D, int GSHIFT, int HPG>
__global__ __launch_bounds__(256 * mass_sets<HPG>(), 1) void dsa_tile_mass_kernel(
    const bf16_t *__restrict__ q, const bf16_t *__restrict__ k, const float *__restrict__ lse,
    const uint32_t *__restrict__ bitmap, int ldw, const int32_t *__restrict__ cu, int N, int T, int Hq, int Hkv,
    float scale_log2, int K, int ngroups, float final_mul, float *__restrict__ table) {
    constexpr int NS = mass_sets<HPG>(), HPW = HPG / NS;       // wave sets; kv heads per wave
    constexpr int KS = D / 16, CPR = D / 8, TILE_B = tile_bytes<D>(), NT = 256 * NS;
    constexpr int Gp = 1 << GSHIFT, QBW = (4 * 32) >> GSHIFT;
    constexpr int CH = 32 * HPG * CPR, LOADS = CH / NT;  // 16-byte chunks of one key tile of all HPG heads; per thread
    static_assert(CH % NT == 0 && LOADS >= 1, "every thread stages the same number of chunks");
    extern __shared__ __attribute__((aligned(16))) unsigned char dyn_lds[];   // [HPG][TILE_B] | sums of the second set
    float *const xbuf = reinterpret_cast<float *>(dyn_lds + HPG * TILE_B);

    const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5, j = lane & 31;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wq = wv & 3, set = wv >> 2;                // query quarter of the block; wave set
    LaneOffsets<D> lo;
    lo.init(lane);
    const int G = Hq / Hkv;
    const int grp = blockIdx.x % ngroups, kvh0 = grp * HPG;
    int s0, L, blk;
    // (heaviest block first over the whole batch: 1.21 against 1.37 ms for the segment-by-segment order at 32 768 tokens)
    if (!locate_block_heaviest_first(cu, N, blockIdx.x / ngroups, QBW, s0, L, blk)) return;
    L = min(L, ldw * 32);                               // a bitmap row has ldw words whatever the caller's max_seqlen
    const int qc0 = blk * QBW;
    if (qc0 >= L) return;

    const int r = wq * 32 + j;
    const int qcol = qc0 + (r >> GSHIFT), head = r & (Gp - 1);
    const bool row_ok = qcol < L && head < G;
    const int t = s0 + min(qcol, L - 1);
    const int ntiles = min(qc0 + QBW - 1, L - 1) / 32 + 1;
    const uint32_t *wrow = bitmap + (int64_t)t * ldw;
    float *prow = table + ((int64_t)grp * T + t) * K;
    if (ngroups == 1) {
        // the table is the result itself: slots past a row's selection (rows shorter than K keys) are zero
        for (int qq = 0; qq < QBW && qc0 + qq < L; ++qq) {
            float *zr = table + (int64_t)(s0 + qc0 + qq) * K;
            for (int jj = qc0 + qq + 1 + tid; jj < K; jj += NT) zr[jj] = 0.f;
        }
    }
    u32x4 kst[LOADS];
    // one key row of the group's kv heads is contiguous in memory (HPG * D elements); kv heads past the last one
    // (a short last group) read the last head again and count for nothing (lse = +inf below)
#define MASS_LOAD(TILE)                                                                             \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) {                                            \
        const int c = i * NT + tid;                                                                \
        const int row = c / (HPG * CPR), hh = (c / CPR) % HPG, ch = c % CPR;                       \
        kst[i] = *reinterpret_cast<const u32x4 *>(                                                 \
            k + ((int64_t)(s0 + min((TILE) * 32 + row, L - 1)) * Hkv + min(kvh0 + hh, Hkv - 1)) * D + ch * 8); \
    }
#define MASS_STORE()                                                                                \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) {                                            \
        const int c = i * NT + tid;                                                                \
        const int row = c / (HPG * CPR), hh = (c / CPR) % HPG, ch = c % CPR;                       \
        *reinterpret_cast<u32x4 *>(&dyn_lds[hh * TILE_B + tile_off<D>(row, ch)]) = kst[i];         \
    }
    MASS_LOAD(0)
    bf16x8 qB[HPW][KS];
    float lse2[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int kv_rel = set * HPW + hh;
        const int kvh = min(kvh0 + kv_rel, Hkv - 1);
        const int hq = kvh * G + min(head, G - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qB[hh][ks] = row_ok ? load_bf16x8(q + ((int64_t)t * Hq + hq) * D + 16 * ks + 8 * h) : zero_bf16x8();
        // padding rows (head >= G, query past the segment, kv head past the last) get lse = +inf: their P is
        // exp2(-inf) = 0 in the sums.  Keys that are not selected need no masking: their sums are never stored.
        const float lse_row = lse[(int64_t)hq * T + t];
        lse2[hh] = (row_ok && kvh0 + kv_rel < Hkv) ? lse_row * LOG2E_F : INFINITY;
    }
    uint32_t word_next = qcol < L ? wrow[0] : 0u;
    int seen = 0;                                        // selected keys of this row in the tiles already walked
    MASS_STORE()
    __syncthreads();
    for (int it = 0; it < ntiles; ++it) {
        MASS_LOAD(min(it + 1, ntiles - 1))               // lands during this tile's matrix work
        const uint32_t word_full = word_next;
        { const uint32_t wl = wrow[min(it + 1, ntiles - 1)]; word_next = qcol < L ? wl : 0u; }
        float p[16];
#pragma unroll
        for (int vi = 0; vi < 16; ++vi) p[vi] = 0.f;
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            // (issuing the matrix work of head hh+1 between the exponentials of head hh in a hand-fixed order
            // measured no faster than what the scheduler makes of this loop)
            const unsigned char *kt = dyn_lds + (set * HPW + hh) * TILE_B;
            f32x16 sacc = zero16();
            constexpr int KH = KS >= 8 ? KS / 2 : KS;    // K operands in flight: half a tile row (registers are short here)
#pragma unroll
            for (int k0 = 0; k0 < KS; k0 += KH) {
                bf16x8 ka[KH];
#pragma unroll
                for (int ks = 0; ks < KH; ++ks) ka[ks] = lo.rowop(kt, k0 + ks);
#pragma unroll
                for (int ks = 0; ks < KH; ++ks) sacc = mfma32(ka[ks], qB[hh][k0 + ks], sacc);
            }
#pragma unroll
            for (int vi = 0; vi < 16; ++vi) p[vi] += fast_exp2(fmaf(sacc[vi], scale_log2, -lse2[hh]));
        }
        if (NS == 2 && set == 1) {                       // the second set's sums: [quarter][element / 4][lane] x 16 bytes
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const f32x4 v4 = {p[4 * c], p[4 * c + 1], p[4 * c + 2], p[4 * c + 3]};
                *reinterpret_cast<f32x4 *>(xbuf + ((wq * 4 + c) * 64 + lane) * 4) = v4;
            }
        }
        __syncthreads();                                 // every wave is done with this tile's K; the sums are in place
        MASS_STORE()
        if (set == 0) {
            if (NS == 2) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const f32x4 v4 = *reinterpret_cast<const f32x4 *>(xbuf + ((wq * 4 + c) * 64 + lane) * 4);
                    p[4 * c] += v4[0]; p[4 * c + 1] += v4[1]; p[4 * c + 2] += v4[2]; p[4 * c + 3] += v4[3];
                }
            }
#pragma unroll
            for (int vi = 0; vi < 16; ++vi) p[vi] = group_sum<GSHIFT>(p[vi]);
            // the lanes of a query share the stores: lane `head` writes the elements vi = u*Gp + head
#pragma unroll
            for (int u = 0; u < 16 / Gp; ++u) {
                float val = p[u * Gp];
#pragma unroll
                for (int g = 1; g < Gp; ++g) val = head == g ? p[u * Gp + g] : val;
                const int vi = u * Gp + head;
                const int bit = 8 * (vi >> 2) + (vi & 3) + 4 * h;    // the key's column in the tile
                if ((word_full >> bit) & 1u) prow[seen + __popc(word_full & ((1u << bit) - 1u))] = val * final_mul;
            }
        }
        seen += __popc(word_full);
        __syncthreads();                                 // the next tile's K is staged; the sums have been read
    }
#undef MASS_LOAD
#undef MASS_STORE
}

// mass[t,j] = inv_hq * sum over the tables of partial[g][t][j] for j < n[t], else 0.  One workgroup per query row
// and blockIdx.y-th part of it, four columns per thread (16-byte accesses when K is a multiple of four).
__global__ __launch_bounds__(256) void dsa_mass_reduce_kernel(const float *__restrict__ partial,
                                                               const int32_t *__restrict__ nsel, int T, int K, int Hkv,
                                                               float inv_hq, float *__restrict__ mass) {
    const int t = blockIdx.x, nt = nsel[t];
    const int64_t row = (int64_t)t * K, plane = (int64_t)T * K;
    if ((K & 3) == 0) {
        for (int j4 = blockIdx.y * 256 + threadIdx.x; j4 < (K >> 2); j4 += gridDim.y * 256) {
            float4 acc = {0.f, 0.f, 0.f, 0.f};
            if (4 * j4 < nt)
                for (int kvh = 0; kvh < Hkv; ++kvh) {
                    const float4 x = *reinterpret_cast<const float4 *>(partial + kvh * plane + row + 4 * j4);
                    acc.x += x.x; acc.y += x.y; acc.z += x.z; acc.w += x.w;
                }
            // slots at and beyond n[t] were never written
            acc.x = 4 * j4 < nt ? acc.x * inv_hq : 0.f;
            acc.y = 4 * j4 + 1 < nt ? acc.y * inv_hq : 0.f;
            acc.z = 4 * j4 + 2 < nt ? acc.z * inv_hq : 0.f;
            acc.w = 4 * j4 + 3 < nt ? acc.w * inv_hq : 0.f;
            *reinterpret_cast<float4 *>(mass + row + 4 * j4) = acc;
        }
    } else {
        for (int jj = blockIdx.y * 256 + threadIdx.x; jj < K; jj += gridDim.y * 256) {
            float acc = 0.f;
            if (jj < nt)
                for (int kvh = 0; kvh < Hkv; ++kvh) acc += partial[kvh * plane + row + jj];
            mass[row + jj] = acc * inv_hq;
        }
    }
}

// ==================================================================================================
// Indexer backward.  The indexer score of a selected pair is  I[t,s] = c * sum_h w[t,h] relu(r[t,h,s]),
// r = q_idx[t,h,:] . k_idx[s,:]  (multi-query attention with ReLU in place of the softmax: Hi heads, one key
// head).  Given dscore[t,j] = dLoss/dI at the selected keys (slot j of key s = its rank in the ascending
// selection list = selected keys of earlier tiles + those below it in the tile's word):
//     G[t,h,s]   = dscore[t,s] * w[t,h] * (r > 0)
//     dq_idx[t,h,:] = c * sum_s G[t,h,s] k_idx[s,:]      dw[t,h] = c * sum_s dscore[t,s] relu(r[t,h,s])
//     dk_idx[s,:]   = c * sum_t sum_h G[t,h,s] q_idx[t,h,:]
// Query side = the dQ walk (rows = (query, indexer head), padded to 32 or 64 rows per query so that the 32
// rows of a wave belong to one query): S^T = K Q^T, G^T on the C layout, dQ^T += K^T G^T.  Key side = the
// key-stationary walk: a wave owns 32 keys (rows in registers) and walks the later queries in blocks of
// 32 heads of one query: S = Q K^T, G on the C layout, dK^T += Q^T G.  Every output row is reduced by one
// wave in a fixed order: deterministic, no atomics.
// ==================================================================================================
template <int D, int GSHIFT, int NW>
__global__ __launch_bounds__(NW * 64, (D <= 128 && NW == 4) ? 2 : 1) void dsa_tile_idxq_kernel(
    const bf16_t *__restrict__ q_idx, const bf16_t *__restrict__ k_idx, const bf16_t *__restrict__ w_idx,
    const float *__restrict__ dscore, const uint32_t *__restrict__ bitmap, int ldw, const int32_t *__restrict__ cu, int N,
    int T, int Hi, int K, float cscale, bf16_t *__restrict__ dq_idx, float *__restrict__ dw) {
    constexpr int KS = D / 16, DT = D / 32, CPR = D / 8, TILE_B = tile_bytes<D>(), LOADS = 32 * CPR / (NW * 64);
    constexpr int NBUF = 2, NT = NW * 64, Gp = 1 << GSHIFT, QBW = (NW * 32) >> GSHIFT;
    static_assert(LOADS >= 1 && GSHIFT >= 5, "a wave's 32 rows are heads of one query");
    __shared__ __attribute__((aligned(16))) unsigned char lds[NBUF][TILE_B];
    __shared__ __attribute__((aligned(16))) float dl_s[NW][32];      // per wave: the gradients of the current tile's 32 keys

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, h = lane >> 5, j = lane & 31;
    LaneOffsets<D> lo;
    lo.init(lane);
    int s0, L, blk;
    if (!LOCATE_QUERY_BLOCK(cu, N, blockIdx.x, QBW, s0, L, blk)) return;
    L = min(L, ldw * 32);
    const int qc0 = blk * QBW;
    if (qc0 >= L) return;
    const int r = wv * 32 + j;
    const int qcol = qc0 + (r >> GSHIFT), head = r & (Gp - 1);
    const bool row_ok = qcol < L && head < Hi;
    const int t = s0 + min(qcol, L - 1), hrow = min(head, Hi - 1);
    u32x4 kst[2][LOADS];
#define IDXQ_LOAD(SET, TILE)                                                                        \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) {                                            \
        const int c = i * NT + tid;                                                                \
        const int row = c / CPR, ch = c % CPR;                                                     \
        kst[SET][i] = *reinterpret_cast<const u32x4 *>(k_idx + (int64_t)(s0 + min((TILE) * 32 + row, L - 1)) * D + ch * 8); \
    }
    IDXQ_LOAD(0, 0)
    bf16x8 qB[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qB[ks] = row_ok ? load_bf16x8(q_idx + ((int64_t)t * Hi + hrow) * D + 16 * ks + 8 * h) : zero_bf16x8();
    const float wrow_v = row_ok ? (float)w_idx[(int64_t)t * Hi + hrow] : 0.f;
    const int ntiles = min(qc0 + QBW - 1, L - 1) / 32 + 1;
    const uint32_t *wrow = bitmap + (int64_t)t * ldw;
    const float *drow = dscore + (int64_t)t * K;
    // selection words run two tiles ahead of the compute and the gradients of a tile's keys one tile ahead: lane j
    // fetches the gradient of key column j of the next tile (both halves of the wave the same)
    uint32_t word_cur = qcol < L ? wrow[0] : 0u, word_nx = qcol < L ? wrow[min(1, ntiles - 1)] : 0u;
    int seen = 0;
    auto fetch_dl = [&](uint32_t word, int before) {
        return drow[min(before + (int)__popc(word & ((1u << j) - 1u)), K - 1)];
    };
    float dl_nx = fetch_dl(word_cur, 0);
    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = zero16();
    float dwacc = 0.f;

#define IDXQ_STORE(SET, BUF, TILE)                                                                  \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) {                                            \
        const int c = i * NT + tid;                                                                \
        const int row = c / CPR, ch = c % CPR;                                                     \
        *reinterpret_cast<u32x4 *>(&lds[BUF][tile_off<D>(row, ch)]) = kst[SET][i];                 \
    }
#define IDXQ_COMPUTE(TILE, BUF)                                                                     \
    {                                                                                              \
        const unsigned char *kt = lds[BUF];                                                        \
        const uint32_t word_full = word_cur;                                                       \
        const float dl = ((word_full >> j) & 1u) ? dl_nx : 0.f;                                    \
        seen += __popc(word_full);                                                                 \
        word_cur = word_nx;                                                                        \
        dl_nx = fetch_dl(word_cur, seen);                /* for the next tile */                   \
        { const uint32_t wl = wrow[min((TILE) + 2, ntiles - 1)]; word_nx = qcol < L ? wl : 0u; }   \
        f32x16 sacc = zero16();                                                                    \
        {                                                                                          \
            bf16x8 ka[KS];                                                                         \
            _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) ka[ks] = lo.rowop(kt, ks);           \
            _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) sacc = mfma32(ka[ks], qB[ks], sacc); \
            sched_reads_ahead<KS, 4, 1>();                                                         \
        }                                                                                          \
        /* the wave's 32 gradients go through its own 128 bytes of LDS: one write and four 16-byte reads per lane     \
           (element vi is key column 8*(vi/4) + 4h + vi%4) instead of sixteen lane permutes */      \
        if (h == 0) dl_s[wv][j] = dl;                                                              \
        float ds[16];                                                                              \
        _Pragma("unroll") for (int g4 = 0; g4 < 4; ++g4) {                                         \
            const f32x4 d4 = *reinterpret_cast<const f32x4 *>(&dl_s[wv][8 * g4 + 4 * h]);          \
            _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                        \
                const float sv = sacc[4 * g4 + e];       /* the row's weight multiplies the finished sum instead */ \
                ds[4 * g4 + e] = sv > 0.f ? d4[e] : 0.f;                                           \
                dwacc = fmaf(ds[4 * g4 + e], sv, dwacc); /* dscore * relu(s) */                     \
            }                                                                                      \
        }                                                                                          \
        const bf16x8 dB0 = pack8(ds), dB1 = pack8(ds + 8);                                         \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) {                                        \
            mfma32_acc(acc[dt], lo.trop(kt, 0, dt), dB0);                                          \
            mfma32_acc(acc[dt], lo.trop(kt, 1, dt), dB1);                                          \
        }                                                                                          \
        sched_reads_ahead<2 * DT, 3, 2>();                                                         \
    }
    TILE_PIPELINE(ntiles, IDXQ_LOAD, IDXQ_STORE, IDXQ_COMPUTE)
#undef IDXQ_LOAD
#undef IDXQ_STORE
#undef IDXQ_COMPUTE

    const float dwt = half_sum_f(dwacc);
    if (row_ok) {
        bf16_t *op = dq_idx + ((int64_t)t * Hi + hrow) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) store_c_tile(op + dt * 32, acc[dt], cscale * wrow_v, h);
        if (h == 0) dw[(int64_t)t * Hi + hrow] = dwt * cscale;
    }
}

// key side.  Workgroup = 4 waves x 32 keys = one 128-key tile of a segment; step b of its walk = all heads
// (HB blocks of 32) of query L-1-b: from the end of the segment down to the tile, so that the workgroups of a
// segment that run side by side read the same index-query rows at about the same time and share them in L2.
template <int D, int GSHIFT>
__global__ __launch_bounds__(256) void dsa_tile_idxk_kernel(
    const bf16_t *__restrict__ q_idx, const bf16_t *__restrict__ k_idx, const bf16_t *__restrict__ w_idx,
    const float *__restrict__ dscore, const uint32_t *__restrict__ bitmap, const int32_t *__restrict__ prefix, int ldw,
    const int32_t *__restrict__ cu, int N, int T, int Hi, int K, float cscale, int chunk_steps,
    float *__restrict__ partial) {
    constexpr int KS = D / 16, DT = D / 32, CPR = D / 8, TILE_B = tile_bytes<D>();
    constexpr int NBUF = 2, HB = (1 << GSHIFT) / 32, LOADS = HB * 32 * CPR / 256;
    static_assert(GSHIFT >= 5 && LOADS >= 1, "steps of 32*HB heads of one query");
    __shared__ __attribute__((aligned(16))) unsigned char lds[NBUF][HB][TILE_B];
    __shared__ __attribute__((aligned(16))) float w_s[NBUF][HB * 32];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, h = lane >> 5, j = lane & 31;
    LaneOffsets<D> lo;
    lo.init(lane);
    int s0, L, blk;
    if (!locate_block(cu, N, blockIdx.x, 128, false, s0, L, blk)) return;
    L = min(L, ldw * 32);
    if (blk * 128 >= L) return;
    const int c0 = blk * 128, kc = c0 + wv * 32;
    const int mykey = kc + j;
    const bool key_ok = mykey < L;
    const int64_t krow = (int64_t)s0 + min(mykey, L - 1);
    const bool kw_ok = kc < L;                           // the word column of this wave's keys exists
    const int kw = kw_ok ? kc >> 5 : 0;
    bf16x8 kB[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kB[ks] = load_bf16x8(k_idx + krow * D + 16 * ks + 8 * h);
    f32x16 dkacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) dkacc[dt] = zero16();
    // queries L-1 down to c0 can have selected keys of this tile; the walk is cut into pieces of chunk_steps queries
    // (blockIdx.y), each piece leaving a partial sum: a tile at the start of a long segment would otherwise be one
    // long serial walk
    const int st0 = blockIdx.y * chunk_steps, nsteps = min(L - c0 - st0, chunk_steps);
    if (nsteps <= 0) return;

    // selection word and slot base of (query of a step, this wave's key column): fetched two LOAD calls before the
    // LOAD that forms the gradient's address from them (register set s serves the odd steps, set 1 the even ones)
    const int last_step = nsteps - 1;
    auto word_of = [&](int step, uint32_t &wq, int32_t &bq) {
        const int64_t o = (int64_t)(s0 + L - 1 - st0 - min(step, last_step)) * ldw + kw;
        wq = kw_ok ? bitmap[o] : 0u;
        bq = prefix[o];
    };
    uint32_t wordp[2], word0;
    int32_t basep[2], base0;
    word_of(0, word0, base0);
    word_of(1, wordp[0], basep[0]);
    word_of(2, wordp[1], basep[1]);

    u32x4 qst[2][LOADS];
    float dl_st[2] = {0.f, 0.f}, dl_buf[NBUF] = {0.f, 0.f};
    bool sel_st[2] = {false, false};
    uint32_t w_st[2] = {0u, 0u};
#define IDXK_LOAD(SET, STEP)                                                                        \
    {                                                                                              \
        const int rel = (STEP), qc = L - 1 - st0 - rel;                                            \
        _Pragma("unroll") for (int i = 0; i < LOADS; ++i) {                                        \
            const int c = i * 256 + tid;                                                           \
            const int row = c / CPR, ch = c % CPR;       /* row = head, padded to 32*HB */          \
            qst[SET][i] = *reinterpret_cast<const u32x4 *>(q_idx + ((int64_t)(s0 + qc) * Hi + min(row, Hi - 1)) * D + ch * 8); \
        }                                                                                          \
        w_st[SET] = reinterpret_cast<const unsigned short *>(w_idx)[(int64_t)(s0 + qc) * Hi + min(tid & (32 * HB - 1), Hi - 1)]; \
        const uint32_t word = wordp[SET];                                                          \
        const int base = basep[SET];                                                               \
        word_of(rel + 2, wordp[SET], basep[SET]);        /* for this register set's next step */    \
        sel_st[SET] = (word >> j) & 1u;                                                            \
        dl_st[SET] = dscore[(int64_t)(s0 + qc) * K + min(base + (int)__popc(word & ((1u << j) - 1u)), K - 1)]; \
    }
#define IDXK_STORE(SET, BUF, STEP)                                                                  \
    {                                                                                              \
        const u32x4 z4 = {0u, 0u, 0u, 0u};                                                         \
        _Pragma("unroll") for (int i = 0; i < LOADS; ++i) {                                        \
            const int c = i * 256 + tid;                                                           \
            const int row = c / CPR, ch = c % CPR;                                                 \
            /* padded heads are zeroed: they add nothing to dK */                                   \
            *reinterpret_cast<u32x4 *>(&lds[BUF][row >> 5][tile_off<D>(row & 31, ch)]) = row < Hi ? qst[SET][i] : z4; \
        }                                                                                          \
        if (tid < 32 * HB) w_s[BUF][tid] = tid < Hi ? __uint_as_float(w_st[SET] << 16) : 0.f;       \
        dl_buf[BUF] = sel_st[SET] ? dl_st[SET] : 0.f;                                              \
    }
#define IDXK_COMPUTE(STEP, BUF)                                                                     \
    {                                                                                              \
        const float dl = dl_buf[BUF];                    /* gradient of (query of the step, this lane's key) */ \
        _Pragma("unroll") for (int hb = 0; hb < HB; ++hb) {                                        \
            const unsigned char *qt = lds[BUF][hb];                                                \
            f32x16 sacc = zero16();                                                                \
            {                                                                                      \
                bf16x8 qa[KS];                                                                     \
                _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) qa[ks] = lo.rowop(qt, ks);       \
                _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) sacc = mfma32(qa[ks], kB[ks], sacc); \
            }                                                                                      \
            float gs[16];                                                                          \
            _Pragma("unroll") for (int g4 = 0; g4 < 4; ++g4) {                                     \
                const f32x4 w4 = *reinterpret_cast<const f32x4 *>(&w_s[BUF][hb * 32 + 8 * g4 + 4 * h]); \
                _Pragma("unroll") for (int e = 0; e < 4; ++e) gs[4 * g4 + e] = sacc[4 * g4 + e] > 0.f ? dl * w4[e] : 0.f; \
            }                                                                                      \
            const bf16x8 gB0 = pack8(gs), gB1 = pack8(gs + 8);                                     \
            _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) {                                    \
                mfma32_acc(dkacc[dt], lo.trop(qt, 0, dt), gB0);                                    \
                mfma32_acc(dkacc[dt], lo.trop(qt, 1, dt), gB1);                                    \
            }                                                                                      \
        }                                                                                          \
    }
    {                                                    // step 0 into register set 0, with the words fetched above
        const uint32_t w1 = wordp[0];
        const int32_t b1 = basep[0];
        wordp[0] = word0;
        basep[0] = base0;
        IDXK_LOAD(0, -2 + 2)                             /* consumes (word0, base0); its own prefetch is overwritten below */
        wordp[0] = w1;
        basep[0] = b1;
    }
    TILE_PIPELINE(nsteps, IDXK_LOAD, IDXK_STORE, IDXK_COMPUTE)
#undef IDXK_LOAD
#undef IDXK_STORE
#undef IDXK_COMPUTE

    if (key_ok) {
        float *pk = partial + ((int64_t)blockIdx.y * T + krow) * D + 4 * h;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const f32x4 o4 = {dkacc[dt][4 * g4] * cscale, dkacc[dt][4 * g4 + 1] * cscale, dkacc[dt][4 * g4 + 2] * cscale,
                                  dkacc[dt][4 * g4 + 3] * cscale};
                *reinterpret_cast<f32x4 *>(pk + dt * 32 + 8 * g4) = o4;
            }
    }
}

// dk_idx[s,:] = sum of the partial sums of the pieces of its tile's walk, in piece order
__global__ __launch_bounds__(256) void dsa_idxk_reduce_kernel(const float *__restrict__ partial,
                                                               const int32_t *__restrict__ cu, int N, int T, int D,
                                                               int chunk_steps, int max_cols, bf16_t *__restrict__ dk_idx) {
    const int s = blockIdx.x * (256 / 32) + (threadIdx.x >> 5), c4 = (threadIdx.x & 31) * 4;   // 32 threads x 4 columns per pass
    if (s >= T) return;
    const int seg = find_segment(cu, N, s);
    const int s0 = cu[seg], L = min(cu[seg + 1] - s0, max_cols);     // as the walk: no column past the bitmap row
    const int c0 = ((s - s0) >> 7) << 7;
    if (c0 >= L) return;
    const int pieces = (L - c0 + chunk_steps - 1) / chunk_steps;
    for (int c = c4; c < D; c += 128) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int pc = 0; pc < pieces; ++pc) acc += *reinterpret_cast<const f32x4 *>(partial + ((int64_t)pc * T + s) * D + c);
        const u32x2 o = {pack2bf(acc[0], acc[1]), pack2bf(acc[2], acc[3])};
        *reinterpret_cast<u32x2 *>(dk_idx + (int64_t)s * D + c) = o;
    }
}

// prefix[t][w] = selected keys of query t in the words before w (the slot of the first selected key of word w)
__global__ __launch_bounds__(64) void dsa_bitmap_prefix_kernel(const uint32_t *__restrict__ bitmap, int ldw,
                                                                int32_t *__restrict__ prefix) {
    const int lane = threadIdx.x;
    const uint32_t *row = bitmap + (int64_t)blockIdx.x * ldw;
    int32_t *orow = prefix + (int64_t)blockIdx.x * ldw;
    int carry = 0;
    for (int w0 = 0; w0 < ldw; w0 += 64) {
        const int w = w0 + lane;
        const int c = w < ldw ? (int)__popc(row[w]) : 0;
        int incl = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int u = __shfl_up(incl, off, 64);
            if (lane >= off) incl += u;
        }
        if (w < ldw) orow[w] = carry + incl - c;
        carry += __shfl(incl, 63, 64);
    }
}

// ==================================================================================================
// dQ: query-stationary, same walk as the forward.
//   S^T = K Q^T, dP^T = V dO^T  (A = K / V tiles row-wise, B = Q^T / dO^T in registers)
//   dS^T = P^T * (dP^T - delta)  on the C layout
//   dQ^T[d,row] += K^T[d,key] dS^T[key,row]   (A = K tile transposed, B = dS^T from the C layout)
// ==================================================================================================
template <int D, bool HAS_IDX, int GSHIFT, int NW>
__global__ __launch_bounds__(NW * 64, (D <= 128 && NW == 4) ? 2 : 1) void dsa_tile_dq_kernel(
    const bf16_t *__restrict__ dout, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, const float *__restrict__ lse, const float *delta,
    const uint32_t *__restrict__ bitmap, int ldw, const int32_t *__restrict__ cu, int N, int T, int Hq, int Hkv,
    float scale, int pos_split, int causal, bf16_t *__restrict__ dq, const bf16_t *__restrict__ out_for_delta,
    float *delta_out) {
    constexpr int KS = D / 16, DT = D / 32, CPR = D / 8, TILE_B = tile_bytes<D>();
    constexpr int NBUF = (D > 128) ? 1 : 2;
    constexpr int NT = NW * 64, Gp = 1 << GSHIFT, QBW = (NW * 32) >> GSHIFT;
    constexpr int CH = 32 * CPR, LOADS = (CH + NT - 1) / NT;   // 16-byte chunks per matrix; per thread (head_dim 96: not all threads)
    static_assert(CH % 64 == 0, "whole waves stage or do not");
    __shared__ __attribute__((aligned(16))) unsigned char lds[NBUF][2][TILE_B];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, h = lane >> 5, j = lane & 31;
    LaneOffsets<D> lo;
    lo.init(lane);
    const int G = Hq / Hkv;
    const int kvh = blockIdx.x % Hkv;
    int s0, L, blk;
    if (!LOCATE_QUERY_BLOCK(cu, N, blockIdx.x / Hkv, QBW, s0, L, blk)) return;
    if (HAS_IDX) L = min(L, ldw * 32);                  // a bitmap row has ldw words whatever the caller's max_seqlen
    const int qc0 = blk * QBW;
    if (qc0 >= pos_split || qc0 >= L) return;

    const int r = wv * 32 + j;
    const int qcol = qc0 + (r >> GSHIFT), head = r & (Gp - 1);
    const bool row_ok = qcol < L && head < G;
    const int t = s0 + min(qcol, L - 1), hq = kvh * G + min(head, G - 1);
    const float scale_log2 = scale * LOG2E_F;
    u32x4 kst[2][LOADS], vst[2][LOADS];
#define DQ_LOAD(SET, TILE)                                                                          \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) if (CH % NT == 0 || i * NT + tid < CH) {     \
        const int c = i * NT + tid;                                                               \
        const int row = c / CPR, ch = c % CPR;                                                     \
        const int64_t off = ((int64_t)(s0 + min((TILE) * 32 + row, L - 1)) * Hkv + kvh) * D + ch * 8; \
        kst[SET][i] = *reinterpret_cast<const u32x4 *>(k + off);                                   \
        vst[SET][i] = *reinterpret_cast<const u32x4 *>(v + off);                                   \
    }
    DQ_LOAD(0, 0)                                       // ahead of the q / dO rows: staging waits for this tile only
    bf16x8 qB[KS], doB[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int64_t off = ((int64_t)t * Hq + hq) * D + 16 * ks + 8 * h;
        qB[ks] = row_ok ? load_bf16x8(q + off) : zero_bf16x8();
        doB[ks] = row_ok ? load_bf16x8(dout + off) : zero_bf16x8();
    }
    // the two accumulators of a tile start from -lse/scale and -delta of the lane's row, so that S - lse/scale and
    // dP - delta come out of the MFMAs (one multiply per element instead of a multiply-add and a subtraction)
    const float neg_lse = -lse[(int64_t)hq * T + t] / scale;
    // delta = rowsum(dO * O) of the lane's row: read, or - when every query row of the launch belongs to this kernel -
    // formed here from the dO row the lane already holds and written out for the key-side pass (one launch and one
    // pass over dO and O less)
    float dlt;
    if (out_for_delta) {                                 // (kernel argument: the same for every wave)
        // the order of dsa_bwd_delta_kernel, so that both give the same bits: chain j of this lane covers the 8-element
        // chunks 2*ks+h with ks = j, j+8, ... (that kernel's lane 2*j+h), then its butterfly over 16 lanes - the three
        // steps between lanes of one parity here, the last one across the lane pair
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            p[j] = 0.f;
#pragma unroll
            for (int ks = j; ks < KS; ks += 8) {
                const int64_t off = ((int64_t)t * Hq + hq) * D + 16 * ks + 8 * h;
                const bf16x8 o8 = row_ok ? load_bf16x8(out_for_delta + off) : zero_bf16x8();
                p[j] = dot8_chain(doB[ks], o8, p[j]);
            }
        }
        const float part = ((p[0] + p[4]) + (p[2] + p[6])) + ((p[1] + p[5]) + (p[3] + p[7]));
        dlt = half_sum_f(part);
        if (row_ok && h == 0) delta_out[(int64_t)hq * T + t] = dlt;
    } else {
        dlt = delta[(int64_t)hq * T + t];
    }
    const float neg_dlt = -dlt;
    const int ntiles = (causal ? min(qc0 + QBW - 1, L - 1) : L - 1) / 32 + 1;
    const int klim = causal ? qcol : L - 1;             // last key column this row may attend (dense mode)
    const uint32_t *wrow = bitmap + (int64_t)t * ldw;

    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = zero16();
    uint32_t word_next = HAS_IDX ? wrow[0] : 0u;        // unconditional loads; rows that are not live are masked at use

#define DQ_STORE(SET, BUF, TILE)                                                                         \
    _Pragma("unroll") for (int i = 0; i < LOADS; ++i) if (CH % NT == 0 || i * NT + tid < CH) {     \
        const int c = i * NT + tid;                                                               \
        const int row = c / CPR, ch = c % CPR;                                                     \
        *reinterpret_cast<u32x4 *>(&lds[BUF][0][tile_off<D>(row, ch)]) = kst[SET][i];              \
        *reinterpret_cast<u32x4 *>(&lds[BUF][1][tile_off<D>(row, ch)]) = vst[SET][i];              \
    }
#define DQ_COMPUTE(TILE, BUF)                                                                       \
    {                                                                                              \
        const int kc0 = (TILE) * 32;                                                               \
        const unsigned char *kt = lds[BUF][0], *vt = lds[BUF][1];                                  \
        uint32_t word = row_ok ? word_next : 0u;                                                   \
        if (HAS_IDX) word_next = wrow[min((TILE) + 1, ntiles - 1)];                                \
        if (!HAS_IDX) word = row_ok ? causal_bits(klim - kc0) : 0u;                                \
        word >>= 4 * h;                                                                            \
        f32x16 sacc, pacc;                                                                         \
        _Pragma("unroll") for (int vi = 0; vi < 16; ++vi) { sacc[vi] = neg_lse; pacc[vi] = neg_dlt; } \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                        \
            sacc = mfma32(lo.rowop(kt, ks), qB[ks], sacc);                              \
            pacc = mfma32(lo.rowop(vt, ks), doB[ks], pacc);                             \
        }                                                                                          \
        sched_reads_ahead<2 * KS, 4, 1>();                                                         \
        float ds[16];                                                                              \
        /* tiles in which every live row keeps all 32 keys skip the mask arithmetic */             \
        if (__builtin_amdgcn_ballot_w64(row_ok && (word & 0x0f0f0f0fu) != 0x0f0f0f0fu) == 0ull) {     \
            _Pragma("unroll") for (int vi = 0; vi < 16; ++vi) ds[vi] = fast_exp2(sacc[vi] * scale_log2) * pacc[vi]; \
        } else {                                                                                   \
            _Pragma("unroll") for (int vi = 0; vi < 16; ++vi) {                                    \
                const float x = keep_or_neginf(sacc[vi] * scale_log2,                              \
                                               bit_mask(word, 8 * (vi >> 2) + (vi & 3)));          \
                ds[vi] = fast_exp2(x) * pacc[vi];                                                  \
            }                                                                                      \
        }                                                                                          \
        const bf16x8 dB0 = pack8(ds), dB1 = pack8(ds + 8);                                         \
        _Pragma("unroll") for (int dt = 0; dt < DT; ++dt) {                                        \
            mfma32_acc(acc[dt], lo.trop(kt, 0, dt), dB0);                           \
            mfma32_acc(acc[dt], lo.trop(kt, 1, dt), dB1);                      \
        }                                                                                          \
        sched_reads_ahead<2 * DT, 3, 2>();                                                         \
    }
    TILE_PIPELINE(ntiles, DQ_LOAD, DQ_STORE, DQ_COMPUTE)
#undef DQ_LOAD
#undef DQ_STORE
#undef DQ_COMPUTE

    if (row_ok) {
        bf16_t *op = dq + ((int64_t)t * Hq + hq) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) store_c_tile(op + dt * 32, acc[dt], scale, h);
    }
}

// ==================================================================================================
// Launch order of the key-stationary workgroups.  A key tile's walk is as long as the part of its segment
// behind it, and the hardware starts workgroups in grid order: handed out segment by segment, the long
// walks of a late long segment start late and the launch ends on them.  This kernel (one workgroup) lists
// the 128-key tiles of all segments longest walk first -
//   mode 0: by the number of tiles behind them, across segments (best balance; for launches of a few rounds
//           of workgroups),
//   mode 1: the segments by length, each one's tiles together (workgroups that run side by side then walk the
//           same q / dO rows and share them in L2, which is worth more than the balance once a launch runs
//           for many rounds),
//   mode 2: as mode 0, and long walks cut into pieces of `pb` steps (a step = `qb` queries), for launches with
//           fewer workgroups than a few rounds of the chip: a launch then ends with its longest walk, however
//           few the workgroups.  A tile in pieces leaves one fp32 partial dK / dV per piece, added in piece
//           order by dsa_dkv_pieces_reduce_kernel.  Walks are cut only if the longest is more than twice the
//           steps a CU gets in a balanced launch (all walks x `wg_per_tile` workgroups / 256); pb = the largest
//           power of two up to half of that (at least 32), doubled until at most `item_cap` entries and
//           `slot_cap` partial slots are needed; it depends on cu_seqlens and these parameters only.
// Table:
//   order[0] = number of entries (or -1: too many segments or tiles for the table, use the plain order),
//   order[1] = pb (0: no walk is cut), order[2] = number of tiles that are cut,
//   order[4 + 4 s .. 7 + 4 s] = segment, tile, piece, first partial slot of the tile (-1: not cut) of entry s,
//   behind the `cap` entries: the entry of the first piece of every cut tile.
// The pieces of a tile are counted from the walk's length bound 128 r / qb of its rank r (tiles behind it,
// itself included); a tile whose own walk is shorter leaves its last pieces empty (the kernels and the
// reduction count the pieces from the walk itself).
// The order changes the schedule only; every tile is still reduced in a fixed order.
// ==================================================================================================
#define DSA_ORDER_MAX_SEGS 4096
#define DSA_ORDER_MAX_TILES 8192                         // tiles of the longest segment
#define DSA_ORDER_EXTRA 4096                             // entries beyond one per tile (pieces)
#define DSA_ORDER_SPLIT_MAX_TILES 1024                   // mode 2: one thread per rank
static_assert(DSA_ORDER_MAX_TILES + 1 >= 2 * DSA_ORDER_MAX_SEGS, "the rank tables of the by-segment order share cnt[]");
__device__ __forceinline__ void order_entry(int32_t *order, int slot, int seg, int tile, int piece, int mslot) {
    *reinterpret_cast<int4 *>(order + 4 + 4 * slot) = make_int4(seg, tile, piece, mslot);
}
__global__ __launch_bounds__(1024) void dsa_tile_order_kernel(const int32_t *__restrict__ cu, int N, int cap, int mode, int qb,
                                                              int wg_per_tile, int item_cap, int slot_cap,
                                                              int32_t *__restrict__ order) {
    __shared__ int nt[DSA_ORDER_MAX_SEGS];               // tiles per segment
    __shared__ int cnt[DSA_ORDER_MAX_TILES + 1];         // cnt[r]: segments with at least r tiles; then: slots before rank r
    __shared__ int part[1024];
    __shared__ unsigned long long part64[16];
    __shared__ int maxnt_s, sum_a, sum_b;
    const int tid = threadIdx.x;
    if (N > DSA_ORDER_MAX_SEGS) {
        if (tid == 0) { order[0] = -1; order[1] = 0; order[2] = 0; }
        return;
    }
    if (tid == 0) { maxnt_s = 0; order[1] = 0; order[2] = 0; }
    __syncthreads();
    int mx = 0;
    for (int i = tid; i < N; i += 1024) {
        const int L = cu[i + 1] - cu[i];
        nt[i] = L > 0 ? (L + 127) / 128 : 0;
        mx = max(mx, nt[i]);
    }
    atomicMax(&maxnt_s, mx);
    __syncthreads();
    const int maxnt = maxnt_s;
    if (maxnt > DSA_ORDER_MAX_TILES) {
        if (tid == 0) order[0] = -1;
        return;
    }
    if (mode == 1) {
        // rank of a segment = segments that are longer, or as long and earlier; cnt[rank] = segment, then its first slot
        int *seg_of = cnt, *first = cnt + DSA_ORDER_MAX_SEGS;     // (both fit: DSA_ORDER_MAX_TILES + 1 >= 2 * DSA_ORDER_MAX_SEGS)
        for (int i = tid; i < N; i += 1024) {
            int rk = 0;
            for (int o = 0; o < N; ++o) rk += nt[o] > nt[i] || (nt[o] == nt[i] && o < i);
            seg_of[rk] = i;
        }
        __syncthreads();
        if (tid == 0) {                                  // N <= 4096 additions
            int run = 0;
            for (int rk = 0; rk < N; ++rk) {
                first[rk] = run;
                run += nt[seg_of[rk]];
            }
            maxnt_s = run;
        }
        __syncthreads();
        const int total = maxnt_s;
        if (total > cap) {
            if (tid == 0) order[0] = -1;
            return;
        }
        if (tid == 0) order[0] = total;
        for (int rk = 0; rk < N; ++rk) {
            const int seg = seg_of[rk], f = first[rk];
            for (int j = tid; j < nt[seg]; j += 1024) order_entry(order, f + j, seg, j, 0, -1);
        }
        return;
    }
    for (int r = 1 + tid; r <= maxnt; r += 1024) {
        int c = 0;
        for (int i = 0; i < N; ++i) c += nt[i] >= r;
        cnt[r] = c;
    }
    __syncthreads();
    if (mode == 2 && maxnt <= DSA_ORDER_SPLIT_MAX_TILES) {
        // thread tid owns rank r = maxnt - tid; pieces of a tile of rank r: ceil((128 r / qb) / pb)
        const int r = maxnt - tid;
        const int c = r >= 1 ? cnt[r] : 0, steps = r >= 1 ? r * (128 / qb) : 0;
        // steps of all walks against the longest one: with `ideal` steps per CU in a balanced launch, walks are cut
        // only if the longest is more than twice that (below, the pieces' own cost - a pipeline fill each, fp32 partial
        // sums written and read back - outweighs the balance), into pieces of about half of it
        if (tid == 0) sum_a = 0;
        __syncthreads();
        if (c) atomicAdd(&sum_a, c * steps);
        __syncthreads();
        const int longest = maxnt * (128 / qb);
        const int ideal = (int)(((int64_t)sum_a * wg_per_tile + 255) / 256);
        __syncthreads();
        int pb = 32;
        while (2 * pb <= ideal / 2) pb <<= 1;            // the largest power of two up to ideal / 2, at least 32
        if (longest <= 2 * ideal) pb = 1 << 30;
        for (;; pb <<= 1) {
            const int np = (steps + pb - 1) / pb;
            if (tid == 0) { sum_a = 0; sum_b = 0; }
            __syncthreads();
            if (c) {
                atomicAdd(&sum_a, c * np);
                if (np > 1) atomicAdd(&sum_b, c * np);
            }
            __syncthreads();
            const bool fits = sum_a <= item_cap && sum_a <= cap && sum_b <= slot_cap;
            const bool whole = pb >= longest;                     // no walk is cut any more
            __syncthreads();
            if (fits || whole) break;
        }
        const int np = (steps + pb - 1) / pb, items = c * np, mults = np > 1 ? c * np : 0;
        // entries, partial slots and cut tiles of the larger ranks: one scan over the triple (21 bits each of a 64-bit
        // word: the caps keep every sum below 2^21)
        const unsigned long long mine = (unsigned long long)items | ((unsigned long long)mults << 21) | ((unsigned long long)(np > 1 ? c : 0) << 42);
        unsigned long long incl = mine;                  // inclusive scan: inside the wave by lane shifts, then over the 16 waves
        const int ln = tid & 63, wvi = tid >> 6;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const unsigned int lo32 = __shfl_up((unsigned int)incl, d, 64), hi32 = __shfl_up((unsigned int)(incl >> 32), d, 64);
            if (ln >= d) incl += (unsigned long long)lo32 | ((unsigned long long)hi32 << 32);
        }
        if (ln == 63) part64[wvi] = incl;
        __syncthreads();
        unsigned long long wave_before = 0ull, all = 0ull;
        for (int w2 = 0; w2 < 16; ++w2) {
            const unsigned long long t2 = part64[w2];
            if (w2 < wvi) wave_before += t2;
            all += t2;
        }
        const unsigned long long excl = wave_before + incl - mine;
        const int before[3] = {(int)(excl & 0x1fffffull), (int)((excl >> 21) & 0x1fffffull), (int)(excl >> 42)};
        const int total = (int)(all & 0x1fffffull);
        if (total > cap || total > item_cap) {           // (only when even whole walks do not fit)
            if (tid == 0) order[0] = -1;
            return;
        }
        if (tid == 0) { order[0] = total; order[1] = pb >= longest ? 0 : pb; order[2] = (int)(all >> 42); }
        if (c) {
            int slot = before[0], ms = before[1], mt = before[2];
            int32_t *cut = order + 4 + 4 * cap;          // entries of the first pieces of the cut tiles, for the reduction
            for (int i = 0; i < N; ++i)
                if (nt[i] >= r) {
                    if (np > 1) cut[mt++] = slot;
                    for (int pc = 0; pc < np; ++pc) order_entry(order, slot++, i, nt[i] - r, pc, np > 1 ? ms : -1);
                    if (np > 1) ms += np;
                }
        }
        return;
    }
    // slots before rank r = sum of cnt[r'] over r' > r: ranks are cut into 1024 runs (run t = the ranks
    // maxnt - t per .. downwards), a scan over the runs' sums, then each thread finishes its run
    const int per = (maxnt + 1023) / 1024;
    int sum = 0;
    for (int u = 0; u < per; ++u) {
        const int r = maxnt - (tid * per + u);
        if (r >= 1) sum += cnt[r];
    }
    part[tid] = sum;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const int add = tid >= d ? part[tid - d] : 0;
        __syncthreads();
        part[tid] += add;
        __syncthreads();
    }
    int before = part[tid] - sum;                        // slots of the runs with larger ranks
    const int total = part[1023];
    __syncthreads();
    for (int u = 0; u < per; ++u) {
        const int r = maxnt - (tid * per + u);
        if (r >= 1) {
            const int c = cnt[r];
            cnt[r] = before;
            before += c;
        }
    }
    __syncthreads();
    if (total > cap) {
        if (tid == 0) order[0] = -1;
        return;
    }
    if (tid == 0) order[0] = total;
    for (int r = 1 + tid; r <= maxnt; r += 1024) {
        int slot = cnt[r];
        for (int i = 0; i < N; ++i)
            if (nt[i] >= r) order_entry(order, slot++, i, nt[i] - r, 0, -1);
    }
}
static inline int order_entries_cap(int T) { return T / 128 + DSA_ORDER_MAX_SEGS + 1 + DSA_ORDER_EXTRA; }
extern "C" size_t dsa_tile_order_bytes(int T) { return ((size_t)order_entries_cap(T) * 5 + 4) * sizeof(int32_t); }
// the tile (and the piece of its walk) of workgroup slot `slot`: from the order table when there is one, else
// segment by segment
__device__ __forceinline__ bool locate_key_tile(const int32_t *order, const int32_t *cu, int N, int slot, int &s0, int &L, int &blk,
                                                int &piece, int &mslot, int &pb) {
    piece = 0;
    mslot = -1;
    pb = 0;
    if (order) {
        const int total = __builtin_amdgcn_readfirstlane(order[0]);
        if (total >= 0) {
            if (slot >= total) return false;
            // (every lane reads the same words; the lane reads tell the compiler that the results are wave-uniform)
            const int4 e = *reinterpret_cast<const int4 *>(order + 4 + 4 * slot);
            const int seg = min(max(__builtin_amdgcn_readfirstlane(e.x), 0), N - 1);
            blk = __builtin_amdgcn_readfirstlane(e.y);
            piece = max(__builtin_amdgcn_readfirstlane(e.z), 0);
            mslot = __builtin_amdgcn_readfirstlane(e.w);
            pb = max(__builtin_amdgcn_readfirstlane(order[1]), 0);
            s0 = __builtin_amdgcn_readfirstlane(cu[seg]);
            L = __builtin_amdgcn_readfirstlane(cu[seg + 1]) - s0;
            return blk >= 0;
        }
    }
    return locate_block(cu, N, slot, 128, false, s0, L, blk);
}
// A walk of `nblocks` steps (block nblocks-1-b at step b, `QB` queries each, the queries q0 .. Lq-1) cut into pieces
// of `pb` steps: narrows q0, Lq and nblocks to piece `piece` and returns the number of pieces (1: the whole walk,
// 0: this piece is empty).  Block boundaries stay where they are, so a piece's blocks are the walk's own.
__device__ __forceinline__ int walk_piece(int pb, int piece, int QB, int &q0, int &Lq, int &nblocks) {
    if (pb <= 0 || nblocks <= pb) return piece == 0 ? 1 : 0;
    const int np = (nblocks + pb - 1) / pb;
    if (piece >= np) return 0;
    const int b_lo = piece * pb, b_hi = min(b_lo + pb, nblocks);
    if (b_lo > 0) Lq = q0 + (nblocks - b_lo) * QB;
    q0 += (nblocks - b_hi) * QB;
    nblocks = b_hi - b_lo;
    return np;
}
// one 32-column d-tile of a C-layout accumulator as fp32 (lane = row j; a lane holds the four columns
// 8*g4 + 4*h + {0..3} of every group g4)
__device__ __forceinline__ void store_c_tile_f32(float *row_dt, const f32x16 &acc, int h) {
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
        const f32x4 w = {acc[4 * g4], acc[4 * g4 + 1], acc[4 * g4 + 2], acc[4 * g4 + 3]};
        *reinterpret_cast<f32x4 *>(row_dt + 8 * g4 + 4 * h) = w;
    }
}
// fp32 partial dK / dV of piece `piece` of a tile in pieces: [slot][kv head][dK | dV][128 keys][D]
__device__ __forceinline__ float *piece_partial(float *partial, int mslot, int piece, int Hkv, int kvh, int D) {
    return partial + ((int64_t)(mslot + piece) * Hkv + kvh) * (2 * 128 * (int64_t)D);
}
// Adds the pieces of every tile that was cut, in piece order, and writes its dK (times the softmax scale) and dV
// rows.  Grid: (cut tiles at most, kv heads, DSA_PIECES_Z slices of a tile's rows).
#define DSA_PIECES_Z 4
__global__ __launch_bounds__(256) void dsa_dkv_pieces_reduce_kernel(const int32_t *__restrict__ order, int cap,
                                                                    const float *__restrict__ partial, const int32_t *__restrict__ cu,
                                                                    int N, int Hkv, int D, int qb, int seq_clamp, float scale,
                                                                    bf16_t *__restrict__ dk, bf16_t *__restrict__ dv) {
    if ((int)blockIdx.x >= __builtin_amdgcn_readfirstlane(order[2])) return;
    const int entry = __builtin_amdgcn_readfirstlane(order[4 + 4 * cap + blockIdx.x]);
    int s0, L, blk, piece, mslot, pb;
    if (!locate_key_tile(order, cu, N, entry, s0, L, blk, piece, mslot, pb)) return;
    if (piece != 0 || mslot < 0 || pb <= 0) return;
    L = min(L, seq_clamp);
    const int c0 = blk * 128;
    if (c0 >= L) return;
    const int nblocks = (L - c0 + qb - 1) / qb;          // (pieces only exist for causal launches: the walk starts at the tile)
    if (nblocks <= pb) return;                           // (its walk fits one piece after all: piece 0 wrote the rows itself)
    const int np = (nblocks + pb - 1) / pb, kvh = blockIdx.y;
    const int keys = min(128, L - c0), cpr = D / 4;      // 16-byte chunks per row
    const int64_t slot_f = 2 * 128 * (int64_t)D;         // floats per (slot, kv head)
    const float *base = partial + ((int64_t)mslot * Hkv + kvh) * slot_f;
    constexpr int U = 4;                                 // independent chunks per thread and pass
    const int chunks = 2 * keys * cpr;                   // dK rows, then dV rows
    for (int c0_ = (blockIdx.z * 256 + threadIdx.x) * U; c0_ < chunks; c0_ += DSA_PIECES_Z * 256 * U) {
        f32x4 acc[U];
        int64_t off[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = min(c0_ + u, chunks - 1);
            const int m = c / (keys * cpr), rest = c % (keys * cpr);
            off[u] = ((int64_t)m * 128 + rest / cpr) * D + (rest % cpr) * 4;
            acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        for (int pc = 0; pc < np; pc += 2) {             // piece order: the sum does not depend on the schedule
            const bool two = pc + 1 < np;
            const float *src0 = base + (int64_t)pc * Hkv * slot_f, *src1 = base + (int64_t)(two ? pc + 1 : pc) * Hkv * slot_f;
            f32x4 x0[U], x1[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                x0[u] = *reinterpret_cast<const f32x4 *>(src0 + off[u]);
                x1[u] = *reinterpret_cast<const f32x4 *>(src1 + off[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                acc[u] += x0[u];
                if (two) acc[u] += x1[u];
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0_ + u;
            if (c < chunks) {
                const int m = c / (keys * cpr), rest = c % (keys * cpr);
                const float mul = m ? 1.f : scale;
                bf16_t *outp = m ? dv : dk;
                uint32_t *dst = reinterpret_cast<uint32_t *>(outp + ((int64_t)(s0 + c0 + rest / cpr) * Hkv + kvh) * D + (rest % cpr) * 4);
                dst[0] = pack2bf(acc[u][0] * mul, acc[u][1] * mul);
                dst[1] = pack2bf(acc[u][2] * mul, acc[u][3] * mul);
            }
        }
    }
}

// ==================================================================================================
// dK, dV for head_dim 256, producer/consumer form, key-stationary ("scatter by key": every key row is
// reduced by one wave, in a fixed query order - or, when the launch cuts the walk into pieces, by one wave per
// piece and a sum over the pieces in piece order - so the result needs no atomics and is bit-reproducible).
// A workgroup owns a 128-key tile (4 groups of 32 keys) of one segment and kv head and
// walks the later queries in blocks of 32 (query, head) rows, from the end of the segment down to the key
// tile: workgroups that run side by side then read the same q / dO rows at about the same time and share
// them in L2.
//   waves 0-3 (producers, one per key group): S = Q K^T and dP = dO V^T against the group's K / V rows
//     held in registers (128 of them), then P and dS = P * (dP - delta) in bf16, written to LDS in MFMA B
//     layout.
//   waves 4-7 (consumers, one per key group): dV^T += dO^T P and dK^T += Q^T dS for block b-1,
//     A operands read transposed from the staged q / dO block, B operands read back from LDS.  They
//     also do all the staging (global -> registers -> LDS one block ahead).
// A consumer's accumulators for all of head_dim would fill 256 registers, so a workgroup covers one half
// of head_dim (`dhalf`, the low bit of its index: the consumers accumulate and write that half, the producers
// repeat S and dP: 48 instead of 32 MFMAs per 32x32 block pair and half).
// LDS (dynamic, ~158 KiB): q/dO blocks in a ring of three, P/dS (and, for blocks of large probabilities,
// the bf16 rounding remainder of P) in a ring of two, row statistics and selection words in a ring of
// three.  One barrier per block.  (head_dim <= 128 runs dsa_tile_dkv2_kernel below.)
// ==================================================================================================
template <int D, bool HAS_IDX, int GSHIFT>
__global__ __launch_bounds__(512, 1) void dsa_tile_dkvpc_kernel(
    const bf16_t *__restrict__ dout, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, const float *__restrict__ lse, const float *__restrict__ delta,
    const uint32_t *__restrict__ bitmap, int ldw, const int32_t *__restrict__ cu, int N, int T, int Hq, int Hkv,
    float scale, int causal, const int32_t *__restrict__ order, float *__restrict__ partial, bf16_t *__restrict__ dk,
    bf16_t *__restrict__ dv) {
    static_assert(D == 256, "head_dim <= 128 runs dsa_tile_dkv2_kernel");
    constexpr int KS = D / 16, DT = D / 32, CPR = D / 8, TILE_B = tile_bytes<D>();
    constexpr int NQD = 3, LEAD = 1;                     // q/dO ring slots; blocks staged ahead of the producers
    constexpr int DTC = DT / 2;                          // d-tiles of one half of head_dim
    // the two halves of head_dim are neighbours in the grid, so that the longest walks of both start in the first round
    const int dhalf = blockIdx.x & 1, bx = blockIdx.x >> 1;
    const int dt0 = dhalf * DTC;
    constexpr int NCHUNK = 32 * CPR;                     // 16-byte chunks per staged operand
    constexpr int CPT = NCHUNK / 256;                    // chunks per consumer thread and operand
    constexpr int Gp = 1 << GSHIFT, QB = 32 >> GSHIFT;
    constexpr int QD_SLOT = 2 * TILE_B;                  // q block | dO block
    // 4 key groups x {P (rows 0-15 | 16-31), dS (same), rounding remainder of P (same)} x 64 lanes x 16 B
    constexpr int PD_GROUP = 6 * 1024, PD_SLOT = 4 * PD_GROUP;
    constexpr int AUX_SLOT = (32 + 32 + 4 * 32) * 4;     // lse | delta | selection words [key group][query]
    static_assert(CPT >= 1 && NCHUNK % 256 == 0, "every consumer thread stages whole chunks");
    extern __shared__ __attribute__((aligned(16))) unsigned char dyn_lds[];
    unsigned char *const qd_ring = dyn_lds;                          // NQD slots
    unsigned char *const pd_ring = dyn_lds + NQD * QD_SLOT;          // 2 slots
    unsigned char *const aux_ring = pd_ring + 2 * PD_SLOT;           // NQD slots
    uint32_t *const split_flag = reinterpret_cast<uint32_t *>(aux_ring + NQD * AUX_SLOT);   // [P/dS slot][key group]
    auto qslot = [](int b) { return b % 3; };

    const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5, j = lane & 31;
    LaneOffsets<D> lo;
    lo.init(lane);
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);         // wave-uniform for the compiler too
    const int kg = wv & 3;
    const bool consumer = wv >= 4;
    const int G = Hq / Hkv;
    const int kvh = bx % Hkv;
    int s0, L, blk, piece, mslot, pb;
    if (!locate_key_tile(order, cu, N, bx / Hkv, s0, L, blk, piece, mslot, pb)) return;
    if (HAS_IDX) L = min(L, ldw * 32);                  // a bitmap row has ldw words whatever the caller's max_seqlen
    if (blk * 128 >= L) return;                         // (whole workgroup, before its first barrier)
    const int c0 = blk * 128, kc = c0 + kg * 32;
    const int mykey = kc + j;
    const bool key_ok = mykey < L;
    const int64_t krow = (int64_t)(s0 + min(mykey, L - 1)) * Hkv + kvh;
    const float scale_log2 = scale * LOG2E_F;
    // the walk: queries q0 .. Lq-1 in nblocks steps - all queries that can see this key tile, or one piece of them
    int q0_ = causal ? c0 : 0, Lq_ = L, nblocks_ = (L - q0_ + QB - 1) / QB;
    const int npieces = walk_piece((causal && partial && mslot >= 0) ? pb : 0, piece, QB, q0_, Lq_, nblocks_);
    if (npieces == 0) return;
    const int q0 = q0_, Lq = Lq_, nblocks = nblocks_;

    if (consumer) {
        // ================= consumers: stage block b+2, then dV^T, dK^T of block b-1 =================
        const int ctid = tid - 256;
        const uint32_t *aux_base;
        int aux_q = 0, aux_stride = 1;
        bool aux_mask_ok = false;
        if (ctid < 64) {                                 // 0..31: lse of row ctid, 32..63: delta of row ctid-32
            const int row = ctid & 31;
            const int hd = min(row & (Gp - 1), G - 1);
            aux_q = row >> GSHIFT;
            aux_base = reinterpret_cast<const uint32_t *>((ctid < 32 ? lse : delta) + (int64_t)(kvh * G + hd) * T + s0);
        } else if (HAS_IDX && ctid < 64 + 4 * QB) {      // selection word of (key group w, query qi)
            const int w = (ctid - 64) / QB;
            aux_q = (ctid - 64) % QB;
            aux_stride = ldw;
            aux_mask_ok = (c0 >> 5) + w < ldw;
            aux_base = bitmap + (int64_t)s0 * ldw + (aux_mask_ok ? (c0 >> 5) + w : 0);
        } else {
            aux_base = reinterpret_cast<const uint32_t *>(lse);
        }
        // Per-thread element offsets of block 0 and what the last block adds to them (its rows past the
        // segment end re-read row L-1); in between a block moves every address by the same stride, so
        // the loop does no index arithmetic per row.
        const int last = nblocks - 1;
        const int64_t blk_bytes = (int64_t)QB * Hq * D * 2;
        const unsigned char *qp[CPT], *dp[CPT];          // this thread's chunks of the block loaded last
        int64_t dlast[CPT];
        int lds_off[CPT];
        bool row_dead_last[CPT], head_ok[CPT];
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int c = i * 256 + ctid, srow = c / CPR, sch = c % CPR;
            const int hd = min(srow & (Gp - 1), G - 1);
            const int qr = srow >> GSHIFT;
            const int over = max(q0 + last * QB + qr - (Lq - 1), 0);     // rows past the end in the last block
            const int64_t off = ((int64_t)(s0 + q0 + last * QB + qr - over) * Hq + kvh * G + hd) * D + sch * 8;
            qp[i] = reinterpret_cast<const unsigned char *>(q + off);
            dp[i] = reinterpret_cast<const unsigned char *>(dout + off);
            dlast[i] = -(int64_t)over * Hq * D * 2;
            row_dead_last[i] = over > 0;
            head_ok[i] = (srow & (Gp - 1)) < G;
            lds_off[i] = tile_off<D>(srow, sch);
        }
        const int64_t aux_blk_bytes = (int64_t)aux_stride * QB * 4;
        const int aux_over = max(q0 + last * QB + aux_q - (Lq - 1), 0);
        const int64_t aux_dlast = -(int64_t)aux_stride * aux_over * 4;
        const unsigned char *ap =
            reinterpret_cast<const unsigned char *>(aux_base + (int64_t)aux_stride * (q0 + last * QB + aux_q - aux_over));
        // one register set (four chunks per operand and thread): a global load has one block-time to land
        u32x4 qst0[CPT], dost0[CPT];
        uint32_t aux_st0;
        // loads the block of step b (block last - b), called with b = 0, 1, 2, ... in turn; past step
        // `last` it reads block 0 again
        auto gload = [&](int b, u32x4 (&qst)[CPT], u32x4 (&dost)[CPT], uint32_t &aux_st) {
            if (b >= 1 && b <= last) {
#pragma unroll
                for (int i = 0; i < CPT; ++i) { qp[i] -= blk_bytes; dp[i] -= blk_bytes; }
                ap -= aux_blk_bytes;
                if (b == 1) {                            // leaving the last block: undo its row clamp
#pragma unroll
                    for (int i = 0; i < CPT; ++i) { qp[i] -= dlast[i]; dp[i] -= dlast[i]; }
                    ap -= aux_dlast;
                }
            }
#pragma unroll
            for (int i = 0; i < CPT; ++i) {
                qst[i] = *reinterpret_cast<const u32x4 *>(qp[i]);
                dost[i] = *reinterpret_cast<const u32x4 *>(dp[i]);
            }
            aux_st = *reinterpret_cast<const uint32_t *>(ap);
        };
        auto lstore = [&](int b, const u32x4 (&qst)[CPT], const u32x4 (&dost)[CPT], uint32_t aux_st) {   // step b -> ring slot b % 3
            unsigned char *slot = qd_ring + qslot(b) * QD_SLOT;
            float *lse_s = reinterpret_cast<float *>(aux_ring + qslot(b) * AUX_SLOT);
            float *dlt_s = lse_s + 32;
            uint32_t *mask_s = reinterpret_cast<uint32_t *>(dlt_s + 32);
            // rows past the segment (last block only) and padded heads are zeroed: they add nothing to dK, dV
            const bool tail = b == 0 || b > last;
#pragma unroll
            for (int i = 0; i < CPT; ++i) {
                u32x4 qv = qst[i], dv4 = dost[i];
                if (tail || G != Gp) {
                    const bool live = head_ok[i] && !(b > last || (b == 0 && row_dead_last[i]));
                    const u32x4 z4 = {0u, 0u, 0u, 0u};
                    qv = live ? qv : z4;
                    dv4 = live ? dv4 : z4;
                }
                *reinterpret_cast<u32x4 *>(slot + lds_off[i]) = qv;
                *reinterpret_cast<u32x4 *>(slot + TILE_B + lds_off[i]) = dv4;
            }
            // a row that is not live (past the segment, past the walk, a padded head) has q = dO = 0 but would read a
            // live row's lse: with lse far below zero its P = exp(0 - lse) overflows and 0 * inf reaches dK and dV.  It gets
            // an lse that makes P vanish instead.
            const bool row_dead = b > last || (b == 0 && aux_over > 0) || ((ctid & 31) & (Gp - 1)) >= G;
            if (ctid < 32) lse_s[ctid] = row_dead ? 1e30f : __uint_as_float(aux_st) * LOG2E_F;
            else if (ctid < 64) dlt_s[ctid - 32] = row_dead ? 0.f : __uint_as_float(aux_st);
            else if (HAS_IDX && ctid < 64 + 4 * QB)
                mask_s[((ctid - 64) / QB) * 32 + (ctid - 64) % QB] =
                    (aux_mask_ok && !(b > last || (b == 0 && aux_over > 0))) ? aux_st : 0u;
        };
        gload(0, qst0, dost0, aux_st0);
        lstore(0, qst0, dost0, aux_st0);
        gload(1, qst0, dost0, aux_st0);
        __syncthreads();                                 // the first step staged

        f32x16 dkacc[DTC], dvacc[DTC];
#pragma unroll
        for (int dt = 0; dt < DTC; ++dt) { dkacc[dt] = zero16(); dvacc[dt] = zero16(); }
        auto consume = [&](int b) {
            const unsigned char *qt = qd_ring + qslot(b) * QD_SLOT + dt0 * 64;
            lds_u8 *pt[4];                  // lane addresses in the q block; the dO block sits TILE_B behind
#pragma unroll
            for (int vv = 0; vv < 4; ++vv) {
                pt[vv] = (lds_u8 *)qt + lo.tr[vv];
                asm volatile("" : "+v"(pt[vv]));         // keep "address + immediate" reads: no re-association
            }
            const unsigned char *pd = pd_ring + (b & 1) * PD_SLOT + kg * PD_GROUP + lane * 16;
            const bf16x8 pB0 = *reinterpret_cast<const bf16x8 *>(pd), pB1 = *reinterpret_cast<const bf16x8 *>(pd + 1024);
            const bf16x8 dB0 = *reinterpret_cast<const bf16x8 *>(pd + 2048), dB1 = *reinterpret_cast<const bf16x8 *>(pd + 3072);
#pragma unroll
            for (int dt = 0; dt < DTC; ++dt) {
                dvacc[dt] = mfma32(LaneOffsets<D>::trop_at(pt, 0, dt, TILE_B), pB0, dvacc[dt]);
                dkacc[dt] = mfma32(LaneOffsets<D>::trop_at(pt, 0, dt, 0), dB0, dkacc[dt]);
                dvacc[dt] = mfma32(LaneOffsets<D>::trop_at(pt, 1, dt, TILE_B), pB1, dvacc[dt]);
                dkacc[dt] = mfma32(LaneOffsets<D>::trop_at(pt, 1, dt, 0), dB1, dkacc[dt]);
            }
            sched_reads_ahead<4 * DTC, 3, 2, 4>();
            // blocks that hold a large probability also carry what bf16 rounded off P (see store_pd): dV += dO^T P_lo
            if (__builtin_amdgcn_readfirstlane(split_flag[(b & 1) * 4 + kg])) {
                const bf16x8 pL0 = *reinterpret_cast<const bf16x8 *>(pd + 4096), pL1 = *reinterpret_cast<const bf16x8 *>(pd + 5120);
#pragma unroll
                for (int dt = 0; dt < DTC; ++dt) {
                    dvacc[dt] = mfma32(LaneOffsets<D>::trop_at(pt, 0, dt, TILE_B), pL0, dvacc[dt]);
                    dvacc[dt] = mfma32(LaneOffsets<D>::trop_at(pt, 1, dt, TILE_B), pL1, dvacc[dt]);
                }
            }
        };
        // one consumer step: stage step b+1 from the register set, refill the set with step b+2, then the MFMAs of step b-1
        for (int b = 0; b <= nblocks; ++b) {
            lstore(b + LEAD, qst0, dost0, aux_st0);      // its slot was last read (as step b+1-3) before the previous barrier
            gload(b + LEAD + 1, qst0, dost0, aux_st0);
            if (b >= 1) consume(b - 1);
            __syncthreads();
        }
        if (npieces > 1) {                               // a piece of the walk: fp32 partial sums, added by the reduction
            float *pk = piece_partial(partial, mslot, piece, Hkv, kvh, D) + (kg * 32 + j) * D + dt0 * 32, *pv_ = pk + 128 * D;
#pragma unroll
            for (int dt = 0; dt < DTC; ++dt) {
                store_c_tile_f32(pk + dt * 32, dkacc[dt], h);
                store_c_tile_f32(pv_ + dt * 32, dvacc[dt], h);
            }
        } else if (key_ok) {
            bf16_t *pk = dk + krow * D + dt0 * 32, *pv_ = dv + krow * D + dt0 * 32;
#pragma unroll
            for (int dt = 0; dt < DTC; ++dt) {
                store_c_tile(pk + dt * 32, dkacc[dt], scale, h);
                store_c_tile(pv_ + dt * 32, dvacc[dt], 1.f, h);
            }
        }
        return;
    }

    // ================= producers: S and dP of a block, then its softmax =================
    bf16x8 kB[KS], vB[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        kB[ks] = load_bf16x8(k + krow * D + 16 * ks + 8 * h);
        vB[ks] = load_bf16x8(v + krow * D + 16 * ks + 8 * h);
    }
    // P and dS go to the consumers in bf16.  dV[s] = sum over (query, head) of P dO piles the rounding of P (2^-9
    // relative) onto one key row; where probabilities are large (few keys per query: short rows, small top-k) and many
    // rows meet in one key, that noise reaches several 1e-2.  A block whose largest P is at least DKV_SPLIT_MIN
    // therefore also carries P - bf16(P), and the consumers add dO^T times it; blocks of small probabilities (the bulk of
    // any long row) skip both the arithmetic and the extra MFMAs.
    constexpr float DKV_SPLIT_MIN = 0.015625f;
    auto store_pd = [&](int b, const float *pv, const float *dsv) {  // -> ring slot b % 2, MFMA B layout
        unsigned char *pd = pd_ring + (b & 1) * PD_SLOT + kg * PD_GROUP + lane * 16;
        const bf16x8 p0 = pack8(pv), p1 = pack8(pv + 8);
        *reinterpret_cast<bf16x8 *>(pd) = p0;
        *reinterpret_cast<bf16x8 *>(pd + 1024) = p1;
        *reinterpret_cast<bf16x8 *>(pd + 2048) = pack8(dsv);
        *reinterpret_cast<bf16x8 *>(pd + 3072) = pack8(dsv + 8);
        float pm = pv[0];
#pragma unroll
        for (int vi = 1; vi < 16; ++vi) pm = fmaxf(pm, pv[vi]);
        const bool big = __builtin_amdgcn_ballot_w64(pm >= DKV_SPLIT_MIN) != 0ull;   // wave-uniform
        if (big) {
            const u32x4 w0 = __builtin_bit_cast(u32x4, p0), w1 = __builtin_bit_cast(u32x4, p1);
            float lo[16];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo[2 * e] = pv[2 * e] - __uint_as_float(w0[e] << 16);
                lo[2 * e + 1] = pv[2 * e + 1] - __uint_as_float(w0[e] & 0xffff0000u);
                lo[8 + 2 * e] = pv[8 + 2 * e] - __uint_as_float(w1[e] << 16);
                lo[9 + 2 * e] = pv[9 + 2 * e] - __uint_as_float(w1[e] & 0xffff0000u);
            }
            *reinterpret_cast<bf16x8 *>(pd + 4096) = pack8(lo);
            *reinterpret_cast<bf16x8 *>(pd + 5120) = pack8(lo + 8);
        }
        if (lane == 0) split_flag[(b & 1) * 4 + kg] = big ? 1u : 0u;
    };
    __syncthreads();                                     // the first step staged
    // GEMMs, then softmax, block by block; the row statistics are taken from LDS group by group (the K and V rows
    // leave no registers to hold them across the GEMMs)
    for (int b = 0; b <= nblocks; ++b) {
        if (b < nblocks) {
            const unsigned char *qt = qd_ring + qslot(b) * QD_SLOT, *dot = qt + TILE_B;
            f32x16 sacc = zero16(), pacc = zero16();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                sacc = mfma32(lo.rowop(qt, ks), kB[ks], sacc);
                pacc = mfma32(lo.rowop(dot, ks), vB[ks], pacc);
            }
            sched_reads_ahead<2 * KS, 4, 1>();
            const float *lse_s = reinterpret_cast<const float *>(aux_ring + qslot(b) * AUX_SLOT);
            const float *dlt_s = lse_s + 32;
            const uint32_t *mask_s = reinterpret_cast<const uint32_t *>(dlt_s + 32) + kg * 32;
            const int qcb = q0 + (nblocks - 1 - b) * QB;
            const bool diag = causal && qcb < kc + 32;
            float pv[16], dsv[16];
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const f32x4 l4g = *reinterpret_cast<const f32x4 *>(&lse_s[8 * g4 + 4 * h]);
                const f32x4 d4g = *reinterpret_cast<const f32x4 *>(&dlt_s[8 * g4 + 4 * h]);
                uint32_t keep = 0u;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int vi = 4 * g4 + e, row = 8 * g4 + 4 * h + e;
                    if (e == 0 || GSHIFT < 2) {          // rows of one query share the mask bit
                        const int qi = row >> GSHIFT;
                        uint32_t w = HAS_IDX ? mask_s[qi] : 0xffffffffu;
                        if (diag) w &= causal_bits(qcb + qi - kc);
                        keep = bit_mask(w, j);
                    }
                    const float p = fast_exp2(keep_or_neginf(fmaf(sacc[vi], scale_log2, -l4g[e]), keep));
                    pv[vi] = p;
                    dsv[vi] = p * (pacc[vi] - d4g[e]);
                }
            }
            store_pd(b, pv, dsv);
        }
        __syncthreads();
    }
}
template <int D>
constexpr size_t dkvpc_lds_bytes() {   // three q/dO and row-data slots, two P/dS slots, the split flags
    return 3 * ((size_t)2 * tile_bytes<D>() + (32 + 32 + 4 * 32) * 4) + 2 * (4 * 6 * 1024) + 2 * 4 * 4;
}

// ==================================================================================================
// dK, dV for head_dim <= 128, "two chains" form.  The same key-stationary walk as dsa_tile_dkvpc_kernel
// (a workgroup owns a 128-key tile of one segment and kv head and walks the later queries from the
// segment end down, 32 (query, head) rows per step); the eight waves are split by GEMM chain, so that
// neither P nor dS has to be handed over in full and every wave runs 16 MFMAs per step:
//   waves 0-3 (P chain, one per 32-key group): S = Q K^T against the group's K rows in registers,
//     started from -lse/scale so that P = exp2(S * scale*log2e) needs no subtraction, the selection bit
//     applied before the exponential; dV^T += dO^T P with P going from the C layout of the first GEMM
//     straight into the B operand of the second.  P also goes to LDS in bf16 for the other chain.
//     Step s: S of block s, then the MFMAs of dV for block s-1 with the softmax of block s behind them.
//   waves 4-7 (dS chain): dP = dO V^T against the group's V rows, started from -delta; dS = P (dP - delta)
//     with the bf16 P read back from LDS; dK^T += Q^T dS, dS staying in registers.  Step s: block s-1.
//     These waves also stage the q / dO blocks and the row data (two steps ahead in LDS, two more in
//     registers).
// One barrier per step; block s sits in ring slot s % 4 from step s-2 (staged) to step s+1 (last read),
// P of block s in slot s % 2 of its ring from step s to step s+1.
// Measured on this kernel's instruction mix (no memory traffic): one wave of each chain on a SIMD needs
// about 1270 clocks per step against 1090 for the 32 MFMAs alone; the kernel runs at about 2000.
// ==================================================================================================
template <int D, bool HAS_IDX, int GSHIFT>
__global__ __launch_bounds__(512, 1) void dsa_tile_dkv2_kernel(
    const bf16_t *__restrict__ dout, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k,
    const bf16_t *__restrict__ v, const float *__restrict__ lse, const float *__restrict__ delta,
    const uint32_t *__restrict__ bitmap, int ldw, const int32_t *__restrict__ cu, int N, int T, int Hq, int Hkv,
    float scale, int causal, const int32_t *__restrict__ order, float *__restrict__ partial, bf16_t *__restrict__ dk,
    bf16_t *__restrict__ dv) {
    static_assert(D <= 128, "head_dim 256 runs dsa_tile_dkvpc_kernel");
    constexpr int KS = D / 16, DT = D / 32, CPR = D / 8, TILE_B = tile_bytes<D>();
    constexpr int NCHUNK = 32 * CPR, STG = 256, CPT = (NCHUNK + STG - 1) / STG;
    constexpr bool ALL_STAGE = NCHUNK % STG == 0;        // (head_dim 96: the last chunk of half of the staging threads is spare)
    constexpr int Gp = 1 << GSHIFT, QB = 32 >> GSHIFT;
    constexpr int QD_SLOT = 2 * TILE_B;                  // q block | dO block
    constexpr int P_GROUP = 2 * 1024, P_SLOT = 4 * P_GROUP;   // per key group: P rows 0-15 | 16-31, 64 lanes x 16 B each
    constexpr int AUX_SLOT = (32 + 32 + 4 * 32) * 4;     // lse | delta | selection words [key group][query]
    static_assert(CPT >= 1 && NCHUNK % 64 == 0, "whole waves stage a chunk or do not");
    extern __shared__ __attribute__((aligned(16))) unsigned char dyn_lds[];
    unsigned char *const qd_ring = dyn_lds;                          // 4 slots
    unsigned char *const p_ring = dyn_lds + 4 * QD_SLOT;             // 2 slots
    unsigned char *const aux_ring = p_ring + 2 * P_SLOT;             // 4 slots

    const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5, j = lane & 31;
    LaneOffsets<D> lo;
    lo.init(lane);
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = wv & 3;
    const int G = Hq / Hkv;
    const int kvh = blockIdx.x % Hkv;
    int s0, L, blk, piece, mslot, pb;
    if (!locate_key_tile(order, cu, N, blockIdx.x / Hkv, s0, L, blk, piece, mslot, pb)) return;
    if (HAS_IDX) L = min(L, ldw * 32);
    if (blk * 128 >= L) return;                         // (whole workgroup, before its first barrier)
    const int c0 = blk * 128, kc = c0 + kg * 32;
    const int mykey = kc + j;
    const bool key_ok = mykey < L;
    const int64_t krow = (int64_t)(s0 + min(mykey, L - 1)) * Hkv + kvh;
    const float scale_log2 = scale * LOG2E_F, inv_scale = 1.f / scale;
    // the walk: queries q0 .. Lq-1 in nblocks steps (step s handles block nblocks-1-s) - all queries that can see
    // this key tile, or one piece of them
    int q0_ = causal ? c0 : 0, Lq_ = L, nblocks_ = (L - q0_ + QB - 1) / QB;
    const int npieces = walk_piece((causal && partial && mslot >= 0) ? pb : 0, piece, QB, q0_, Lq_, nblocks_);
    if (npieces == 0) return;
    const int q0 = q0_, Lq = Lq_, nblocks = nblocks_;

    // an accumulator in C layout that starts from a per-row value (lane (key, h) holds rows 8 g4 + 4 h + e)
    auto rows_init = [&](const float *rowv) __attribute__((always_inline)) {
        f32x16 c;
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const f32x4 r = *reinterpret_cast<const f32x4 *>(&rowv[8 * g4 + 4 * h]);
#pragma unroll
            for (int e = 0; e < 4; ++e) c[4 * g4 + e] = r[e];
        }
        return c;
    };
    // Staging: 16-byte chunks of the q and dO blocks, CPT of each per thread, and one word of row data per thread of
    // the first 64 + 4 QB (lse, delta, selection words).  Step b reads block nblocks-1-b; the walk starts at the
    // segment end, so only block 0 (rows past the end) and the steps past the last block need their rows zeroed.
    const int ctid = tid & 255;                          // used by the dS chain's waves
    const int last = nblocks - 1;
    const int64_t blk_bytes = (int64_t)QB * Hq * D * 2;
    const unsigned char *qp[CPT], *dp[CPT];
    int64_t dlast[CPT];
    int lds_off[CPT];
    bool row_dead_last[CPT], head_ok[CPT], staged[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
        staged[i] = ALL_STAGE || i * STG + ctid < NCHUNK; // a spare chunk loads the tile's last chunk again and stores nothing
        const int c = min(i * STG + ctid, NCHUNK - 1), srow = c / CPR, sch = c % CPR;
        const int hd = min(srow & (Gp - 1), G - 1);
        const int qr = srow >> GSHIFT;
        const int over = max(q0 + last * QB + qr - (Lq - 1), 0);     // rows past the end in the last block
        const int64_t off = ((int64_t)(s0 + q0 + last * QB + qr - over) * Hq + kvh * G + hd) * D + sch * 8;
        qp[i] = reinterpret_cast<const unsigned char *>(q + off);
        dp[i] = reinterpret_cast<const unsigned char *>(dout + off);
        dlast[i] = -(int64_t)over * Hq * D * 2;
        row_dead_last[i] = over > 0;
        head_ok[i] = (srow & (Gp - 1)) < G;
        lds_off[i] = tile_off<D>(srow, sch);
    }
    // row data: every thread loads one word and stores one word, threads without a share into a spare LDS word.
    // lse and delta go in as -lse/scale and -delta (the chains start their accumulators from them), selection words
    // as they are (zero for key groups past the bitmap row)
    const uint32_t *aux_base = reinterpret_cast<const uint32_t *>(lse);
    int aux_q = 0, aux_stride = 0, aux_lds = 4 * AUX_SLOT;          // spare word behind the four slots
    float aux_mul = 0.f;
    uint32_t aux_and = 0u;
    bool aux_is_word = false, aux_pad = false;
    uint32_t aux_dead_value = 0u;                    // what a row that is not live stores: word 0, delta 0, -lse/scale -1e30
    if (ctid < 64) {                                 // 0..31: lse of row ctid, 32..63: delta of row ctid-32
        const int row = ctid & 31;
        const int hd = min(row & (Gp - 1), G - 1);
        aux_pad = (row & (Gp - 1)) >= G;
        aux_dead_value = ctid < 32 ? __float_as_uint(-1e30f) : 0u;
        aux_q = row >> GSHIFT;
        aux_stride = 1;
        aux_base = reinterpret_cast<const uint32_t *>((ctid < 32 ? lse : delta) + (int64_t)(kvh * G + hd) * T + s0);
        aux_mul = ctid < 32 ? -inv_scale : -1.f;
        aux_lds = ctid * 4;
    } else if (HAS_IDX && ctid < 64 + 4 * QB) {      // selection word of (key group w, query qi)
        const int w = (ctid - 64) / QB;
        aux_q = (ctid - 64) % QB;
        aux_stride = ldw;
        const bool ok = (c0 >> 5) + w < ldw;
        aux_base = bitmap + (int64_t)s0 * ldw + (ok ? (c0 >> 5) + w : 0);
        aux_and = ok ? 0xffffffffu : 0u;
        aux_is_word = true;
        aux_lds = (64 + w * 32 + aux_q) * 4;
    }
    const int64_t aux_blk_bytes = (int64_t)aux_stride * QB * 4;
    const int aux_over = max(q0 + last * QB + aux_q - (Lq - 1), 0);
    const int64_t aux_dlast = -(int64_t)aux_stride * aux_over * 4;
    const unsigned char *ap =
        reinterpret_cast<const unsigned char *>(aux_base + (int64_t)aux_stride * (q0 + last * QB + aux_q - aux_over));
    u32x4 qst0[CPT], dost0[CPT], qst1[CPT], dost1[CPT];     // two register sets: a load has two steps to land
    uint32_t aux_st0, aux_st1;
    auto aux_value = [&](uint32_t x) __attribute__((always_inline)) {
        return aux_is_word ? (x & aux_and) : __float_as_uint(__uint_as_float(x) * aux_mul);
    };
    // general forms (first and last steps): gload is called with b = 0, 1, 2, ... in turn; past step `last` it reads
    // the first block again and lstore zeroes what it stores
    auto gload = [&](int b, u32x4 (&qst)[CPT], u32x4 (&dost)[CPT], uint32_t &aux_st) __attribute__((always_inline)) {
        if (b >= 1 && b <= last) {
#pragma unroll
            for (int i = 0; i < CPT; ++i) { qp[i] -= blk_bytes; dp[i] -= blk_bytes; }
            ap -= aux_blk_bytes;
            if (b == 1) {                            // leaving the last block: undo its row clamp
#pragma unroll
                for (int i = 0; i < CPT; ++i) { qp[i] -= dlast[i]; dp[i] -= dlast[i]; }
                ap -= aux_dlast;
            }
        }
        aux_st = *reinterpret_cast<const uint32_t *>(ap);   // first: its consumer then never waits for younger loads
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            qst[i] = *reinterpret_cast<const u32x4 *>(qp[i]);
            dost[i] = *reinterpret_cast<const u32x4 *>(dp[i]);
        }
    };
    auto lstore = [&](int b, const u32x4 (&qst)[CPT], const u32x4 (&dost)[CPT], uint32_t aux_st) __attribute__((always_inline)) {
        unsigned char *slot = qd_ring + (b & 3) * QD_SLOT;
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const bool live = head_ok[i] && !(b > last || (b == 0 && row_dead_last[i]));
            const u32x4 z4 = {0u, 0u, 0u, 0u};
            if (ALL_STAGE || staged[i]) {
                *reinterpret_cast<u32x4 *>(slot + lds_off[i]) = live ? qst[i] : z4;
                *reinterpret_cast<u32x4 *>(slot + TILE_B + lds_off[i]) = live ? dost[i] : z4;
            }
        }
        // a row that is not live (past the segment, past the walk, a padded head) has q = dO = 0 but would read a live
        // row's lse: with lse far below zero its P = exp(0 - lse) overflows and 0 * inf reaches dK and dV.  Its selection
        // word is cleared, and its S starts so low that P vanishes also where no selection masks it.
        const bool dead = b > last || (b == 0 && aux_over > 0) || aux_pad;
        *reinterpret_cast<uint32_t *>(aux_ring + (aux_lds < 4 * AUX_SLOT ? (b & 3) * AUX_SLOT : 0) + aux_lds) =
            dead ? aux_dead_value : aux_value(aux_st);
    };
    // steady forms (blocks 2 .. last of a group whose heads fill the padded group): no branch, no select
    auto gload_steady = [&](u32x4 (&qst)[CPT], u32x4 (&dost)[CPT], uint32_t &aux_st) __attribute__((always_inline)) {
        ap -= aux_blk_bytes;
        aux_st = *reinterpret_cast<const uint32_t *>(ap);
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            qp[i] -= blk_bytes;
            dp[i] -= blk_bytes;
            qst[i] = *reinterpret_cast<const u32x4 *>(qp[i]);
            dost[i] = *reinterpret_cast<const u32x4 *>(dp[i]);
        }
    };
    auto lstore_steady = [&](int b, const u32x4 (&qst)[CPT], const u32x4 (&dost)[CPT], uint32_t aux_st) __attribute__((always_inline)) {
        unsigned char *slot = qd_ring + (b & 3) * QD_SLOT;
#pragma unroll
        for (int i = 0; i < CPT; ++i)
            if (ALL_STAGE || staged[i]) {
                *reinterpret_cast<u32x4 *>(slot + lds_off[i]) = qst[i];
                *reinterpret_cast<u32x4 *>(slot + TILE_B + lds_off[i]) = dost[i];
            }
        *reinterpret_cast<uint32_t *>(aux_ring + (aux_lds < 4 * AUX_SLOT ? (b & 3) * AUX_SLOT : 0) + aux_lds) = aux_value(aux_st);
    };
    if (wv >= 4) {
        // ================= dS chain: staging, then dP, dS, dK of the block the P chain finished a step earlier =================
        gload(0, qst0, dost0, aux_st0);
        gload(1, qst1, dost1, aux_st1);
        bf16x8 vB[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) vB[ks] = load_bf16x8(v + krow * D + 16 * ks + 8 * h);
        lstore(0, qst0, dost0, aux_st0);
        lstore(1, qst1, dost1, aux_st1);
        gload(2, qst0, dost0, aux_st0);
        gload(3, qst1, dost1, aux_st1);
        __syncthreads();                                 // steps 0 and 1 staged

        f32x16 dkacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) dkacc[dt] = zero16();
        // dS of elements 8 half .. 8 half + 7 (C layout) as an MFMA B operand: the other chain's bf16 P times this
        // chain's dP - delta
        auto ds_half = [&](const u32x4 &w, const f32x16 &pacc, int half) __attribute__((always_inline)) {
            float ds[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                ds[2 * e] = __uint_as_float(w[e] << 16) * pacc[8 * half + 2 * e];
                ds[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u) * pacc[8 * half + 2 * e + 1];
            }
            return pack8(ds);
        };
        // block b: dP = dO V^T starting from -delta, dS, dK^T += Q^T dS.  Operand reads run three to four MFMAs ahead
        // (every MFMA step ends in an empty asm statement that the next operand passes through, which fixes the
        // order); the second half of dS is formed behind the first MFMAs of dK.
        auto block = [&](int b) __attribute__((always_inline)) {
            const unsigned char *qt = qd_ring + (b & 3) * QD_SLOT, *dot = qt + TILE_B;
            const unsigned char *pd = p_ring + (b & 1) * P_SLOT + kg * P_GROUP + lane * 16;
            f32x16 pacc = rows_init(reinterpret_cast<const float *>(aux_ring + (b & 3) * AUX_SLOT) + 32);
            bf16x8 a[4], t[4];
#pragma unroll
            for (int i = 0; i < 4 && i < KS; ++i) a[i] = lo.rowop(dot, i);
            const u32x4 w0 = *reinterpret_cast<const u32x4 *>(pd), w1 = *reinterpret_cast<const u32x4 *>(pd + 1024);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                pacc = mfma32(a[ks & 3], vB[ks], pacc);
                if (ks + 4 < KS) a[ks & 3] = lo.rowop(dot, ks + 4);
                if (ks + 3 >= KS) t[ks + 3 - KS] = lo.trop(qt, (ks + 3 - KS) / DT, (ks + 3 - KS) % DT);
                if (ks + 1 < KS) asm volatile("" : "+v"(a[(ks + 1) & 3]) : : "memory");
                else asm volatile("" : "+v"(t[0]) : : "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
            const bf16x8 dB0 = ds_half(w0, pacc, 0);
            uint32_t dw[4];
#pragma unroll
            for (int m = 0; m < 2 * DT; ++m) {
                if (m < DT) dkacc[m] = mfma32(t[m & 3], dB0, dkacc[m]);
                else {
                    const u32x4 d1 = {dw[0], dw[1], dw[2], dw[3]};
                    dkacc[m - DT] = mfma32(t[m & 3], __builtin_bit_cast(bf16x8, d1), dkacc[m - DT]);
                }
                if (m + 3 < 2 * DT) t[(m + 3) & 3] = lo.trop(qt, (m + 3) / DT, (m + 3) % DT);
                if (m < DT) {                            // the four pairs of the second half of dS, spread behind these MFMAs
#pragma unroll
                    for (int e = 4 * m / DT; e < 4 * (m + 1) / DT; ++e) {
                        dw[e] = pack2bf(__uint_as_float(w1[e] << 16) * pacc[8 + 2 * e], __uint_as_float(w1[e] & 0xffff0000u) * pacc[9 + 2 * e]);
                        asm volatile("" : "+v"(dw[e]));
                    }
                }
                if (m + 1 < 2 * DT) asm volatile("" : "+v"(t[(m + 1) & 3]) : : "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
        };
#define DKV2_DS_STEP(S, QS, DS_, AS)                                                                \
    {                                                                                              \
        lstore((S) + 2, QS, DS_, AS); /* its slot was last read (as step S-2) before the previous barrier */ \
        gload((S) + 4, QS, DS_, AS);                                                               \
        if ((S) >= 1) block((S) - 1);                                                              \
        __syncthreads();                                                                             \
    }
#define DKV2_DS_STEADY(S, QS, DS_, AS)                                                              \
    {                                                                                              \
        lstore_steady((S) + 2, QS, DS_, AS);                                                       \
        gload_steady(QS, DS_, AS);                                                                 \
        block((S) - 1);                                                                            \
        __syncthreads();                                                                             \
    }
        DKV2_DS_STEP(0, qst0, dost0, aux_st0)
        int s = 1;
        if (s <= nblocks) {
            DKV2_DS_STEP(1, qst1, dost1, aux_st1)
            s = 2;
        }
        if (G == Gp)                                     // steps whose staged block is 2 .. last and whose loaded block is 2 .. last
            for (; s + 5 <= last; s += 2) {
                DKV2_DS_STEADY(s, qst0, dost0, aux_st0)
                DKV2_DS_STEADY(s + 1, qst1, dost1, aux_st1)
            }
        for (; s + 1 <= nblocks; s += 2) {
            DKV2_DS_STEP(s, qst0, dost0, aux_st0)
            DKV2_DS_STEP(s + 1, qst1, dost1, aux_st1)
        }
        if (s <= nblocks) DKV2_DS_STEP(s, qst0, dost0, aux_st0)
#undef DKV2_DS_STEP
#undef DKV2_DS_STEADY
        if (npieces > 1) {                               // a piece of the walk: fp32 partial sums, added by the reduction
            float *pk = piece_partial(partial, mslot, piece, Hkv, kvh, D) + (kg * 32 + j) * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) store_c_tile_f32(pk + dt * 32, dkacc[dt], h);
        } else if (key_ok) {
            bf16_t *pk = dk + krow * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) store_c_tile(pk + dt * 32, dkacc[dt], scale, h);
        }
        return;
    }

    // ================= P chain: S and softmax of block s, dV of block s-1 =================
    bf16x8 kB[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kB[ks] = load_bf16x8(k + krow * D + 16 * ks + 8 * h);
    uint32_t mw[16];
    auto read_aux = [&](int b) __attribute__((always_inline)) {                         // selection words of step b
        const uint32_t *mask_s = reinterpret_cast<const uint32_t *>(aux_ring + (b & 3) * AUX_SLOT) + 64 + kg * 32;
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (HAS_IDX && (e == 0 || GSHIFT < 2)) mw[4 * g4 + e] = mask_s[(8 * g4 + 4 * h + e) >> GSHIFT];
    };
    f32x16 dvacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) dvacc[dt] = zero16();
    // P of element vi (C layout) of step b from its S accumulator (which started from -lse/scale); pm collects the
    // block's largest P
    auto element = [&](auto may_diag, int b, int vi, const f32x16 &sacc, float sl2, uint32_t &keep, float &pm) __attribute__((always_inline)) {
        const int g4 = vi >> 2, e = vi & 3, row = 8 * g4 + 4 * h + e;
        if (e == 0 || GSHIFT < 2) {                      // rows of one query share the mask bit
            const int qcb = q0 + (nblocks - 1 - b) * QB, qi = row >> GSHIFT;
            uint32_t w = HAS_IDX ? mw[vi] : 0xffffffffu;
            if (decltype(may_diag)::value && causal && qcb < kc + 32) w &= causal_bits(qcb + qi - kc);
            keep = bit_mask(w, j);
        }
        const float p = fast_exp2(keep_or_neginf(sacc[vi] * sl2, keep));
        pm = fmaxf(pm, p);
        return p;
    };
    auto store_p = [&](int b, int half, bf16x8 p) __attribute__((always_inline)) {
        *reinterpret_cast<bf16x8 *>(p_ring + (b & 1) * P_SLOT + kg * P_GROUP + half * 1024 + lane * 16) = p;
    };
    // P goes on in bf16.  dV[s] = sum over (query, head) of P dO piles the rounding of P (2^-9 relative) onto one key
    // row; where probabilities are large (few keys per query) and many rows meet in one key, that noise reaches
    // several 1e-2.  A block whose largest P is at least DKV_SPLIT_MIN therefore also adds dO^T (P - bf16(P)).
    constexpr float DKV_SPLIT_MIN = 0.015625f;
    auto remainder = [&](auto may_diag, int b, const f32x16 &sc, float pm, bf16x8 p0, bf16x8 p1) __attribute__((always_inline)) {
        if (__builtin_amdgcn_ballot_w64(pm >= DKV_SPLIT_MIN) != 0ull) {   // wave-uniform, rare: P is formed again
            const u32x4 w0 = __builtin_bit_cast(u32x4, p0), w1 = __builtin_bit_cast(u32x4, p1);
            float pv[16], lo_[16], pm2 = 0.f;
            uint32_t keep = 0u;
#pragma unroll
            for (int vi = 0; vi < 16; ++vi) pv[vi] = element(may_diag, b, vi, sc, scale_log2, keep, pm2);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo_[2 * e] = pv[2 * e] - __uint_as_float(w0[e] << 16);
                lo_[2 * e + 1] = pv[2 * e + 1] - __uint_as_float(w0[e] & 0xffff0000u);
                lo_[8 + 2 * e] = pv[8 + 2 * e] - __uint_as_float(w1[e] << 16);
                lo_[9 + 2 * e] = pv[9 + 2 * e] - __uint_as_float(w1[e] & 0xffff0000u);
            }
            const unsigned char *dot = qd_ring + (b & 3) * QD_SLOT + TILE_B;
            const bf16x8 l0 = pack8(lo_), l1 = pack8(lo_ + 8);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                dvacc[dt] = mfma32(lo.trop(dot, 0, dt), l0, dvacc[dt]);
                dvacc[dt] = mfma32(lo.trop(dot, 1, dt), l1, dvacc[dt]);
            }
        }
    };
    // Step s: S of block s (KS MFMAs), then the 2 DT MFMAs of dV^T += dO^T P of block s-1 with the softmax of
    // 16 / (2 DT) elements of block s behind each of them (operand reads three MFMAs ahead; every MFMA step ends in
    // empty asm statements that its results and the next MFMA's operand pass through, which fixes the order).
    bf16x8 pq0 = zero_bf16x8(), pq1 = zero_bf16x8();     // P of the block before, as B operands (rows 0-15 | 16-31)
    auto step = [&](auto may_diag, auto has_cur, auto has_prev, int s) __attribute__((always_inline)) {
        constexpr bool CUR = decltype(has_cur)::value, PREV = decltype(has_prev)::value;
        constexpr int NM = 2 * DT;                       // elements 16 m / NM .. 16 (m + 1) / NM behind MFMA m
        const unsigned char *qt = qd_ring + (s & 3) * QD_SLOT, *dprev = qd_ring + ((s - 1) & 3) * QD_SLOT + TILE_B;
        f32x16 sacc;
        if (CUR) {
            sacc = rows_init(reinterpret_cast<const float *>(aux_ring + (s & 3) * AUX_SLOT));
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) sacc = mfma32(lo.rowop(qt, ks), kB[ks], sacc);
            sched_reads_ahead<KS, (KS >= 4 ? 4 : KS), 1, 4>();
            __builtin_amdgcn_sched_barrier(0);
        }
        float pv[2], pm = 0.f, sl2 = scale_log2;
        uint32_t keep = 0u, pw[8];
        bf16x8 t[4];
        if (PREV) {
#pragma unroll
            for (int i = 0; i < 3 && i < NM; ++i) t[i] = lo.trop(dprev, i / DT, i % DT);
        }
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            if (PREV) {
                dvacc[m % DT] = mfma32(t[m & 3], m < DT ? pq0 : pq1, dvacc[m % DT]);
                if (m + 3 < NM) t[(m + 3) & 3] = lo.trop(dprev, (m + 3) / DT, (m + 3) % DT);
            }
            if (CUR) {
#pragma unroll
                for (int vi = 16 * m / NM; vi < 16 * (m + 1) / NM; ++vi) {   // P is packed pair by pair as it is formed
                    pv[vi & 1] = element(may_diag, s, vi, sacc, sl2, keep, pm);
                    if (vi & 1) {
                        pw[vi >> 1] = pack2bf(pv[0], pv[1]);
                        asm volatile("" : "+v"(pw[vi >> 1]));
                    } else {
                        asm volatile("" : "+v"(pv[0]));
                    }
                }
            }
            if (PREV && m + 1 < NM) asm volatile("" : "+v"(sl2), "+v"(pm), "+v"(t[(m + 1) & 3]) : : "memory");
            else asm volatile("" : "+v"(sl2), "+v"(pm) : : "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
        if (CUR) {
            const u32x4 w0 = {pw[0], pw[1], pw[2], pw[3]}, w1 = {pw[4], pw[5], pw[6], pw[7]};
            pq0 = __builtin_bit_cast(bf16x8, w0);
            pq1 = __builtin_bit_cast(bf16x8, w1);
            store_p(s, 0, pq0);
            store_p(s, 1, pq1);
            remainder(may_diag, s, sacc, pm, pq0, pq1);
            if (s + 1 < nblocks) read_aux(s + 1);
        }
    };
    const std::true_type yes;
    const std::false_type no;
    __syncthreads();                                     // steps 0 and 1 staged
    read_aux(0);
    // The blocks that can touch the causal diagonal come last; the steady loop before them has no mask
    // arithmetic besides the selection bits.
    const int nb_diag = causal ? max(kc + 32 - q0 + QB - 1, 0) / QB : 0;   // (none for a piece that starts past the diagonal)
    const int steady = max(nblocks - nb_diag, 1);        // steps [1, steady) see blocks fully past the diagonal
    step(yes, yes, no, 0);
    __syncthreads();
    int s = 1;
    for (; s < steady; ++s) {
        step(no, yes, yes, s);
        __syncthreads();
    }
    for (; s < nblocks; ++s) {
        step(yes, yes, yes, s);
        __syncthreads();
    }
    step(yes, no, yes, nblocks);
    __syncthreads();
    if (npieces > 1) {
        float *pv_ = piece_partial(partial, mslot, piece, Hkv, kvh, D) + (128 + kg * 32 + j) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) store_c_tile_f32(pv_ + dt * 32, dvacc[dt], h);
    } else if (key_ok) {
        bf16_t *pv_ = dv + krow * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) store_c_tile(pv_ + dt * 32, dvacc[dt], 1.f, h);
    }
}
template <int D>
constexpr size_t dkv2_lds_bytes() {   // q/dO ring, P ring, row-data ring and one spare word
    return 4 * ((size_t)2 * tile_bytes<D>() + (32 + 32 + 4 * 32) * 4) + 2 * (4 * 2 * 1024) + 16;
}

// ==================================================================================================
// launchers: instantiate per head_dim, mask kind and (power-of-two padded) group size
// ==================================================================================================
static inline int group_shift(int Hq, int Hkv) {
    const int G = Hq / Hkv;
    int gshift = 0;
    while ((1 << gshift) < G) ++gshift;
    return gshift;
}

// waves per workgroup of the query-stationary kernels: all of them share the staged K / V tiles
#ifndef DSA_TILE_WAVES_128
#define DSA_TILE_WAVES_128 8
#endif
template <int D> constexpr int tile_waves() { return (D == 128 || D == 96) ? DSA_TILE_WAVES_128 : 4; }
static inline int tile_waves_of(int D) { return (D == 128 || D == 96) ? DSA_TILE_WAVES_128 : 4; }
template <int D, bool HAS_IDX, int GS>
static hipError_t launch_fwd_i(dim3 grid, hipStream_t stream, const void *q, const void *k, const void *v,
                         const uint32_t *bitmap, int ldw, const int32_t *cu, int N, int T, int Hq, int Hkv, float sl2,
                         int pos_split, int causal, void *out, float *lse) {
    constexpr int NW = tile_waves<D>();
    if constexpr (NW == 8) {
        // A launch of a few rounds of workgroups is bound by what a workgroup pays before its first tile and after
        // its last (memory round trips, row stores), and with eight waves only one workgroup fits a CU.  Such
        // launches run the four-wave form, two workgroups per CU, whose fixed parts overlap (forward -9 % on 8192
        // tokens in seven segments; the dQ kernel measured 19 % slower that way and keeps eight waves).
        if (grid.x <= DSA_BATCH_ORDER_MAX_BLOCKS) {
            const int Gp = 1 << GS;
            const dim3 grid4((unsigned)(((int64_t)T / ((32 * 4) / Gp) + N + 1) * Hkv));
            hipLaunchKernelGGL((dsa_tile_fwd_kernel<D, HAS_IDX, GS, 4>), grid4, dim3(256), 0, stream, (const bf16_t *)q,
                               (const bf16_t *)k, (const bf16_t *)v, bitmap, ldw, cu, N, T, Hq, Hkv, sl2, pos_split, causal, (bf16_t *)out, lse);
            return hipSuccess;
        }
    }
    hipLaunchKernelGGL((dsa_tile_fwd_kernel<D, HAS_IDX, GS, NW>), grid, dim3(64 * NW), 0, stream, (const bf16_t *)q,
                       (const bf16_t *)k, (const bf16_t *)v, bitmap, ldw, cu, N, T, Hq, Hkv, sl2, pos_split, causal, (bf16_t *)out, lse);
    return hipSuccess;
}
template <int D, bool HAS_IDX, int GS>
static hipError_t launch_dq_i(dim3 grid, hipStream_t stream, const void *dout, const void *q, const void *k, const void *v,
                        const float *lse, const float *delta, const uint32_t *bitmap, int ldw, const int32_t *cu, int N,
                        int T, int Hq, int Hkv, float scale, int pos_split, int causal, void *dq, const void *out_for_delta,
                        float *delta_out) {
    hipLaunchKernelGGL((dsa_tile_dq_kernel<D, HAS_IDX, GS, tile_waves<D>()>), grid, dim3(64 * tile_waves<D>()), 0, stream, (const bf16_t *)dout,
                       (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, bitmap, ldw, cu, N, T, Hq, Hkv,
                       scale, pos_split, causal, (bf16_t *)dq, (const bf16_t *)out_for_delta, delta_out);
    return hipSuccess;
}
template <int D, bool HAS_IDX, int GS>
static hipError_t launch_dkv_i(dim3 grid, hipStream_t stream, const void *dout, const void *q, const void *k, const void *v,
                         const float *lse, const float *delta, const uint32_t *bitmap, int ldw, const int32_t *cu, int N,
                         int T, int Hq, int Hkv, float scale, int causal, const int32_t *order, float *partial, void *dk,
                         void *dv) {
    // LDS above 64 KiB has to be requested per kernel and device; asked for on every launch (a host-side table
    // lookup), so that neither a second device nor a second thread can meet a kernel that was never configured
    if constexpr (D <= 128) {
        const hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void *>(&dsa_tile_dkv2_kernel<D, HAS_IDX, GS>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)dkv2_lds_bytes<D>());
        if (e2 != hipSuccess) return e2;
        hipLaunchKernelGGL((dsa_tile_dkv2_kernel<D, HAS_IDX, GS>), grid, dim3(512), dkv2_lds_bytes<D>(), stream,
                           (const bf16_t *)dout, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, bitmap,
                           ldw, cu, N, T, Hq, Hkv, scale, causal, order, partial, (bf16_t *)dk, (bf16_t *)dv);
        return hipSuccess;
    } else {
    const hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void *>(&dsa_tile_dkvpc_kernel<D, HAS_IDX, GS>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)dkvpc_lds_bytes<D>());
    if (ea != hipSuccess) return ea;
    // two workgroups per key tile and kv head, one per half of head_dim (a consumer wave holds 128 accumulator registers)
    hipLaunchKernelGGL((dsa_tile_dkvpc_kernel<D, HAS_IDX, GS>), dim3(grid.x * 2), dim3(512), dkvpc_lds_bytes<D>(), stream,
                       (const bf16_t *)dout, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, lse, delta, bitmap,
                       ldw, cu, N, T, Hq, Hkv, scale, causal, order, partial, (bf16_t *)dk, (bf16_t *)dv);
    return hipSuccess;
    }
}

#define GS_SWITCH(FN, DD, HI, ...)                                    \
    switch (gs) {                                                     \
        case 0: launch_status = FN<DD, HI, 0>(__VA_ARGS__); break;    \
        case 1: launch_status = FN<DD, HI, 1>(__VA_ARGS__); break;    \
        case 2: launch_status = FN<DD, HI, 2>(__VA_ARGS__); break;    \
        case 3: launch_status = FN<DD, HI, 3>(__VA_ARGS__); break;    \
        default: launch_status = FN<DD, HI, 4>(__VA_ARGS__); break;   \
    }
#define TILE_SWITCH(FN, ...)                                                              \
    hipError_t launch_status = hipSuccess;                                                \
    switch (D) {                                                                          \
        case 64: if (bitmap) { GS_SWITCH(FN, 64, true, __VA_ARGS__) } else { GS_SWITCH(FN, 64, false, __VA_ARGS__) } break;    \
        case 128: if (bitmap) { GS_SWITCH(FN, 128, true, __VA_ARGS__) } else { GS_SWITCH(FN, 128, false, __VA_ARGS__) } break; \
        case 256: if (bitmap) { GS_SWITCH(FN, 256, true, __VA_ARGS__) } else { GS_SWITCH(FN, 256, false, __VA_ARGS__) } break; \
        default: return hipErrorInvalidValue;                                             \
    }                                                                                     \
    if (launch_status != hipSuccess) return launch_status;

// the same with head_dim 96 (dense only: no selection bitmap), for the three attention kernels
#define TILE_SWITCH_96(FN, ...)                                                           \
    hipError_t launch_status = hipSuccess;                                                \
    switch (D) {                                                                          \
        case 64: if (bitmap) { GS_SWITCH(FN, 64, true, __VA_ARGS__) } else { GS_SWITCH(FN, 64, false, __VA_ARGS__) } break;    \
        case 96: if (bitmap) return hipErrorInvalidValue; GS_SWITCH(FN, 96, false, __VA_ARGS__) break;                         \
        case 128: if (bitmap) { GS_SWITCH(FN, 128, true, __VA_ARGS__) } else { GS_SWITCH(FN, 128, false, __VA_ARGS__) } break; \
        case 256: if (bitmap) { GS_SWITCH(FN, 256, true, __VA_ARGS__) } else { GS_SWITCH(FN, 256, false, __VA_ARGS__) } break; \
        default: return hipErrorInvalidValue;                                             \
    }                                                                                     \
    if (launch_status != hipSuccess) return launch_status;

extern "C" hipError_t dsa_launch_tile_fwd(const void *q, const void *k, const void *v, const uint32_t *bitmap, int ldw,
                                          const int32_t *cu, int N, int T, int Hq, int Hkv, int D, float scale,
                                          int pos_split, int causal, void *out, float *lse, hipStream_t stream) {
    const int gs = group_shift(Hq, Hkv);
    const dim3 grid((unsigned)(((int64_t)T / ((32 * tile_waves_of(D)) >> gs) + N + 1) * Hkv));
    TILE_SWITCH_96(launch_fwd_i, grid, stream, q, k, v, bitmap, ldw, cu, N, T, Hq, Hkv, scale * LOG2E_F, pos_split, causal, out, lse)
    return hipGetLastError();
}
// kv heads a workgroup of the attention-mass kernel takes (a power of two, at most what its registers hold; with
// one query head per kv head a lane also holds all sixteen sums of a tile to itself, which costs the top size)
template <int D>
static int mass_hpg(int Hq, int Hkv) {
    const int most = Hq == Hkv ? mass_heads_max<D>() / 2 : mass_heads_max<D>();
    int hpg = 1;
    while (hpg * 2 <= most && hpg < Hkv) hpg *= 2;
    return hpg;
}
extern "C" int dsa_mass_groups(int Hq, int Hkv, int D) {
    const int hpg = D == 64 ? mass_hpg<64>(Hq, Hkv) : D == 128 ? mass_hpg<128>(Hq, Hkv) : mass_hpg<256>(Hq, Hkv);
    return (Hkv + hpg - 1) / hpg;
}
template <int D, int GS, int HPG>
static hipError_t launch_mass_h(dim3 grid, hipStream_t stream, const void *q, const void *k, const float *lse,
                                const uint32_t *bitmap, int ldw, const int32_t *cu, int N, int T, int Hq, int Hkv, float sl2,
                                int K, int ngroups, float final_mul, float *table) {
    if constexpr (HPG > mass_heads_max<D>()) {
        return hipErrorInvalidValue;
    } else {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&dsa_tile_mass_kernel<D, GS, HPG>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)mass_lds_bytes<D, HPG>());
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((dsa_tile_mass_kernel<D, GS, HPG>), grid, dim3(256 * mass_sets<HPG>()), (mass_lds_bytes<D, HPG>()), stream,
                           (const bf16_t *)q, (const bf16_t *)k, lse, bitmap, ldw, cu, N, T, Hq, Hkv, sl2, K, ngroups, final_mul,
                           table);
        return hipSuccess;
    }
}
template <int D, bool HAS_IDX, int GS>
static hipError_t launch_mass_i(dim3 grid, hipStream_t stream, const void *q, const void *k, const float *lse,
                          const uint32_t *bitmap, int ldw, const int32_t *cu, int N, int T, int Hq, int Hkv, float sl2,
                          int K, int ngroups, float final_mul, float *table) {
    switch (mass_hpg<D>(Hq, Hkv)) {
        case 1: return launch_mass_h<D, GS, 1>(grid, stream, q, k, lse, bitmap, ldw, cu, N, T, Hq, Hkv, sl2, K, ngroups, final_mul, table);
        case 2: return launch_mass_h<D, GS, 2>(grid, stream, q, k, lse, bitmap, ldw, cu, N, T, Hq, Hkv, sl2, K, ngroups, final_mul, table);
        case 4: return launch_mass_h<D, GS, 4>(grid, stream, q, k, lse, bitmap, ldw, cu, N, T, Hq, Hkv, sl2, K, ngroups, final_mul, table);
        case 8: return launch_mass_h<D, GS, 8>(grid, stream, q, k, lse, bitmap, ldw, cu, N, T, Hq, Hkv, sl2, K, ngroups, final_mul, table);
        default: return launch_mass_h<D, GS, 16>(grid, stream, q, k, lse, bitmap, ldw, cu, N, T, Hq, Hkv, sl2, K, ngroups, final_mul, table);
    }
}
// attention mass of the selected keys: the heads of a query summed in registers, scaled by 1/Hq and written into
// mass (T,K); batches with more kv heads than one workgroup holds leave one (T,K) table per group in `partial`,
// which dsa_mass_reduce_kernel adds in group order
extern "C" hipError_t dsa_launch_tile_mass(const void *q, const void *k, const float *lse, const uint32_t *bitmap,
                                           int ldw, const int32_t *n, const int32_t *cu, int N, int T, int Hq, int Hkv,
                                           int D, int K, float scale, float *partial, float *mass, hipStream_t stream) {
    const int gs = group_shift(Hq, Hkv);
    const int ngroups = dsa_mass_groups(Hq, Hkv, D);
    const dim3 grid((unsigned)(((int64_t)T / ((32 * 4) >> gs) + N + 1) * ngroups));
    const float inv_hq = 1.f / (float)Hq;
    float *table = ngroups == 1 ? mass : partial;
    const float final_mul = ngroups == 1 ? inv_hq : 1.f;
    TILE_SWITCH(launch_mass_i, grid, stream, q, k, lse, bitmap, ldw, cu, N, T, Hq, Hkv, scale * LOG2E_F, K, ngroups, final_mul, table)
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || ngroups == 1) return e;
    const unsigned parts = (unsigned)((K / 4 + 255) / 256 > 0 ? (K / 4 + 255) / 256 : 1);
    hipLaunchKernelGGL(dsa_mass_reduce_kernel, dim3(T, parts < 8 ? parts : 8), dim3(256), 0, stream, partial, n, T, K, ngroups,
                       inv_hq, mass);
    return hipGetLastError();
}
// indexer backward: prefix table, query side (dq_idx, dw), key side (dk_idx).  D = indexer head_dim (64 or 128),
// at most 64 indexer heads.
// Queries per piece of a key tile's walk in the indexer backward.  A piece is one workgroup and about 1.3 us per query:
// the finer the pieces, the better a launch of few thousand of them balances over 512 workgroup slots (32 768 tokens:
// 6.26 -> 5.95 ms with 256 instead of 512, 6.31 with 128; 8192 tokens: 0.44 -> 0.31 -> 0.25 ms), the more fp32 partial
// sums (one (T, Di) plane per piece index).  Depends on T, and on the bound of the longest segment only where the
// planes would pass 1.25 GiB.
static int idxk_chunk(int T, int Di, int ldw) {
    int c = T <= 16384 ? 128 : 256;
    while ((size_t)((ldw * 32 + c - 1) / c) * T * Di * 4 > ((size_t)5 << 28) && c < (1 << 20)) c *= 2;
    return c;
}
template <int D, int GS>
static void launch_idx_bwd_i(hipStream_t stream, const void *q_idx, const void *k_idx, const void *w_idx, const float *dscore,
                             const uint32_t *bitmap, const int32_t *prefix, int ldw, const int32_t *cu, int N, int T, int Hi,
                             int K, float cscale, void *dq_idx, void *dk_idx, float *dw, float *partial, hipStream_t stream_q) {
    constexpr int NW = tile_waves<D>();
    // (the key side, the longer pass, is issued first: with two streams it gets the GPU first)
    const int chunk = idxk_chunk(T, D, ldw);
    const dim3 gk((unsigned)((int64_t)T / 128 + N + 1), (unsigned)((ldw * 32 + chunk - 1) / chunk));
    hipLaunchKernelGGL((dsa_tile_idxk_kernel<D, GS>), gk, dim3(256), 0, stream, (const bf16_t *)q_idx, (const bf16_t *)k_idx,
                       (const bf16_t *)w_idx, dscore, bitmap, prefix, ldw, cu, N, T, Hi, K, cscale, chunk, partial);
    hipLaunchKernelGGL(dsa_idxk_reduce_kernel, dim3((unsigned)((T + 7) / 8)), dim3(256), 0, stream, partial, cu, N, T, D,
                       chunk, ldw * 32, (bf16_t *)dk_idx);
    const dim3 gq((unsigned)((int64_t)T / ((32 * NW) >> GS) + N + 1));
    hipLaunchKernelGGL((dsa_tile_idxq_kernel<D, GS, NW>), gq, dim3(64 * NW), 0, stream_q, (const bf16_t *)q_idx,
                       (const bf16_t *)k_idx, (const bf16_t *)w_idx, dscore, bitmap, ldw, cu, N, T, Hi, K, cscale,
                       (bf16_t *)dq_idx, dw);
}
extern "C" size_t dsa_indexer_bwd_partial_bytes(int T, int Di, int ldw) {
    const int chunk = idxk_chunk(T, Di, ldw);
    return (size_t)((ldw * 32 + chunk - 1) / chunk) * T * Di * 4;
}
extern "C" hipError_t dsa_launch_indexer_bwd(const void *q_idx, const void *k_idx, const void *w_idx, const float *dscore,
                                             const uint32_t *bitmap, int32_t *prefix, int ldw, const int32_t *cu, int N,
                                             int T, int Hi, int Di, int K, float cscale, void *dq_idx, void *dk_idx,
                                             float *dw, float *partial, hipStream_t stream, hipStream_t stream_q) {
    if (Hi < 1 || Hi > 64 || !(Di == 64 || Di == 128)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(dsa_bitmap_prefix_kernel, dim3(T), dim3(64), 0, stream, bitmap, ldw, prefix);
    if (Di == 128) {
        if (Hi > 32) launch_idx_bwd_i<128, 6>(stream, q_idx, k_idx, w_idx, dscore, bitmap, prefix, ldw, cu, N, T, Hi, K, cscale, dq_idx, dk_idx, dw, partial, stream_q);
        else launch_idx_bwd_i<128, 5>(stream, q_idx, k_idx, w_idx, dscore, bitmap, prefix, ldw, cu, N, T, Hi, K, cscale, dq_idx, dk_idx, dw, partial, stream_q);
    } else {
        if (Hi > 32) launch_idx_bwd_i<64, 6>(stream, q_idx, k_idx, w_idx, dscore, bitmap, prefix, ldw, cu, N, T, Hi, K, cscale, dq_idx, dk_idx, dw, partial, stream_q);
        else launch_idx_bwd_i<64, 5>(stream, q_idx, k_idx, w_idx, dscore, bitmap, prefix, ldw, cu, N, T, Hi, K, cscale, dq_idx, dk_idx, dw, partial, stream_q);
    }
    return hipGetLastError();
}
extern "C" hipError_t dsa_launch_tile_dq(const void *dout, const void *q, const void *k, const void *v,
                                         const float *lse, const float *delta, const uint32_t *bitmap, int ldw,
                                         const int32_t *cu, int N, int T, int Hq, int Hkv, int D, float scale,
                                         int pos_split, int causal, void *dq, const void *out_for_delta, float *delta_out,
                                         hipStream_t stream) {
    // out_for_delta != null: the kernel forms delta = rowsum(dO * O) of its rows itself and writes it to delta_out
    const int gs = group_shift(Hq, Hkv);
    const dim3 grid((unsigned)(((int64_t)T / ((32 * tile_waves_of(D)) >> gs) + N + 1) * Hkv));
    TILE_SWITCH_96(launch_dq_i, grid, stream, dout, q, k, v, lse, delta, bitmap, ldw, cu, N, T, Hq, Hkv, scale, pos_split, causal, dq, out_for_delta, delta_out)
    return hipGetLastError();
}
// bytes of fp32 partial sums a launch of T tokens may use for key-tile walks in pieces (0: launches of this size are
// never cut); a slot = the dK and dV of one 128-key tile and kv head
extern "C" size_t dsa_tile_dkv_partial_bytes(int T) {
    if (T <= 0 || T > 131072) return 0;
    const size_t b = (size_t)T * 16384;
    return b < ((size_t)128 << 20) ? b : ((size_t)128 << 20);
}
extern "C" hipError_t dsa_launch_tile_dkv(const void *dout, const void *q, const void *k, const void *v,
                                          const float *lse, const float *delta, const uint32_t *bitmap, int ldw,
                                          const int32_t *cu, int N, int T, int Hq, int Hkv, int D, float scale, int causal,
                                          int32_t *order, float *partial, size_t partial_bytes, void *dk, void *dv,
                                          hipStream_t stream) {
    const int gs = group_shift(Hq, Hkv);
    const int tiles_ub = T / 128 + N;                    // 128-key tiles of all segments, at most
    dim3 grid((unsigned)((tiles_ub + 1) * Hkv));
    // `order` (dsa_tile_order_bytes(T) bytes, or null): the tiles are listed longest walk first before the launch.
    // A launch of at most four workgroups per CU may also cut long walks into pieces (`partial`: fp32 partial sums), so
    // that it does not end on a few long walks with most of the chip idle.
    const int wg_per_tile = Hkv * (D > 128 ? 2 : 1);
    const int64_t slot_pairs = partial ? (int64_t)(partial_bytes / ((size_t)2 * 128 * D * sizeof(float))) : 0;
    const bool pieces = order && causal && slot_pairs >= Hkv && (int64_t)tiles_ub * wg_per_tile <= 4 * 256;
    int item_cap = 0;
    if (order && (N > 1 || pieces)) {
        const int cap = order_entries_cap(T);
        item_cap = pieces ? std::min(cap, tiles_ub + (1024 + wg_per_tile - 1) / wg_per_tile) : cap;
        hipLaunchKernelGGL(dsa_tile_order_kernel, dim3(1), dim3(1024), 0, stream, cu, N, cap,
                           pieces ? 2 : (grid.x > 4 * 256 ? 1 : 0), 32 >> gs, wg_per_tile, item_cap, (int)(slot_pairs / Hkv < (1 << 20) ? slot_pairs / Hkv : (1 << 20)),   /* (sums stay below 2^21) */
                           order);
        if (pieces) grid.x = (unsigned)(item_cap * Hkv);
    } else {
        order = nullptr;                                 // one segment: its tiles are in order already
    }
    if (!pieces) partial = nullptr;
    TILE_SWITCH_96(launch_dkv_i, grid, stream, dout, q, k, v, lse, delta, bitmap, ldw, cu, N, T, Hq, Hkv, scale, causal, order, partial, dk, dv)
    if (pieces)
        hipLaunchKernelGGL(dsa_dkv_pieces_reduce_kernel, dim3(tiles_ub, Hkv, DSA_PIECES_Z), dim3(256), 0, stream, order,
                           order_entries_cap(T), partial, cu, N, Hkv, D, 32 >> gs, bitmap ? ldw * 32 : 0x7fffffff, scale,
                           (bf16_t *)dk, (bf16_t *)dv);
    return hipGetLastError();
}
