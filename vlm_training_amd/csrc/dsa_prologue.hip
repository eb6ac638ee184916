// Pre-attention prologue and post-attention gate of the reference's attention layers, fused:
//   q, k  <-  rope(rms_norm(q_proj), cos, sin)   written straight into the packed (T, H, D) layout the
//             attention operator reads   (models/qwen3_vl/model.py:256-269, models/qwen3_5/model.py:110-129:
//             F.rms_norm per head, transpose, apply_rope, transpose back, .contiguous())
//   out   <-  out * sigmoid(gate)          (models/qwen3_5/model.py:135)
// HBM-bound element-wise work with one reduction per (token, head) row: a row of D bf16 is spread over
// D/8 lanes (16 bytes per lane), so a wave handles 512/D rows per step; the row reduction and the
// rotate_half partner (R/16 lanes away) are cross-lane moves inside those D/8 lanes.  One wave per token
// and step walks the token's query heads, then its key heads; cos/sin of the token are loaded once.
// The backward pass returns the gradients of the projections' outputs and per-workgroup partial sums of
// the two norm weights' gradients (reduced by a second kernel in a fixed order: no atomics).
#include "dsa_common.h"

typedef float f32x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ f32x8 bf8_to_f32(u32x4 w) {
    f32x8 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        r[2 * i] = __uint_as_float(w[i] << 16);
        r[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
    return r;
}
__device__ __forceinline__ u32x4 f32_to_bf8(f32x8 x) {
    return u32x4{pack2bf(x[0], x[1]), pack2bf(x[2], x[3]), pack2bf(x[4], x[5]), pack2bf(x[6], x[7])};
}
__device__ __forceinline__ float bf16_round(float x) { return __uint_as_float(pack2bf(x, 0.f) << 16); }

// cos/sin of this lane's 8 elements of token t (zero-filled past the rotary width R)
template <bool CS_F32>
__device__ __forceinline__ void load_cs(const void *cs, int64_t t, int R, int d0, f32x8 &out, float fill) {
    if (d0 < R) {
        if (CS_F32) {
            const float *p = reinterpret_cast<const float *>(cs) + t * R + d0;
            const f32x4 a = *reinterpret_cast<const f32x4 *>(p), b = *reinterpret_cast<const f32x4 *>(p + 4);
            out = f32x8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
        } else {
            out = bf8_to_f32(*reinterpret_cast<const u32x4 *>(reinterpret_cast<const bf16_t *>(cs) + t * R + d0));
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = fill;
    }
}

// sum over the LPR lanes that share a row (LPR is a power of two <= 32; rows are aligned groups of lanes)
template <int LPR>
__device__ __forceinline__ float row_sum(float x) {
#pragma unroll
    for (int m = 1; m < LPR; m <<= 1) x += __shfl_xor(x, m, 64);
    return x;
}

// a norm weight as the module holds it: fp32 (the trainer's master parameters under autocast) or bf16
__device__ __forceinline__ float norm_weight(const void *w, int w_bf16, int d) {
    return w_bf16 ? (float)reinterpret_cast<const bf16_t *>(w)[d] : reinterpret_cast<const float *>(w)[d];
}

template <int D, bool CS_F32>
__global__ __launch_bounds__(256) void dsa_qk_norm_rope_fwd_kernel(
    const bf16_t *__restrict__ q_in, int64_t q_tok, int64_t q_head, const bf16_t *__restrict__ k_in, int64_t k_tok,
    int64_t k_head, const void *__restrict__ qw, const void *__restrict__ kw, int w_bf16, float eps, float w_offset,
    const void *__restrict__ cosp, const void *__restrict__ sinp, int R, int T, int Hq, int Hkv,
    bf16_t *__restrict__ q_out, bf16_t *__restrict__ k_out, float *__restrict__ q_rstd, float *__restrict__ k_rstd) {
    constexpr int LPR = D / 8, RPW = 64 / LPR;           // lanes per row, rows per wave and step
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int sub = lane / LPR, d0 = (lane % LPR) * 8;
    const int half_lanes = R / 16;                       // rotate_half partner distance in lanes
    const bool low = d0 < R / 2, rot = d0 < R;
    f32x8 wq, wk;
#pragma unroll
    for (int i = 0; i < 8; ++i) { wq[i] = norm_weight(qw, w_bf16, d0 + i) + w_offset; wk[i] = norm_weight(kw, w_bf16, d0 + i) + w_offset; }
    for (int64_t t = (int64_t)blockIdx.x * 4 + wv; t < T; t += (int64_t)gridDim.x * 4) {
        f32x8 c, s;
        load_cs<CS_F32>(cosp, t, R, d0, c, 1.f);
        load_cs<CS_F32>(sinp, t, R, d0, s, 0.f);
        const int H = Hq + Hkv;
        for (int r0 = 0; r0 < H; r0 += RPW) {
            const int r = r0 + sub;
            const bool live = r < H, isq = r < Hq;
            const int hh = live ? (isq ? r : r - Hq) : 0;
            const bf16_t *src = isq ? q_in + t * q_tok + hh * q_head : k_in + t * k_tok + hh * k_head;
            f32x8 x = bf8_to_f32(live ? *reinterpret_cast<const u32x4 *>(src + d0) : u32x4{0u, 0u, 0u, 0u});
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
            const float rstd = rsqrtf(row_sum<LPR>(ss) * (1.f / D) + eps);
            const f32x8 w = isq ? wq : wk;
            f32x8 n, y;
#pragma unroll
            for (int i = 0; i < 8; ++i) n[i] = bf16_round(x[i] * rstd * w[i]);       // F.rms_norm returns bf16
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // rotate_half: element i < R/2 takes -n[i + R/2], element R/2 <= i < R takes n[i - R/2]
                const float other = __shfl(n[i], low ? lane + half_lanes : lane - half_lanes, 64);
                y[i] = rot ? n[i] * c[i] + (low ? -other : other) * s[i] : n[i];
            }
            if (live) {
                bf16_t *dst = isq ? q_out + ((int64_t)t * Hq + hh) * D : k_out + ((int64_t)t * Hkv + hh) * D;
                *reinterpret_cast<u32x4 *>(dst + d0) = f32_to_bf8(y);
                if (d0 == 0) (isq ? q_rstd + (int64_t)t * Hq : k_rstd + (int64_t)t * Hkv)[hh] = rstd;
            }
        }
    }
}

// gradients: g = d(loss)/d(rope output).  dn = rope^T g, dx = rstd * (dn*w - xhat * mean(dn*w*xhat)),
// dw += dn * xhat (per workgroup partial sums: part[block][q|k][D])
template <int D, bool CS_F32>
__global__ __launch_bounds__(256) void dsa_qk_norm_rope_bwd_kernel(
    const bf16_t *__restrict__ gq, const bf16_t *__restrict__ gk, const bf16_t *__restrict__ q_in, int64_t q_tok,
    int64_t q_head, const bf16_t *__restrict__ k_in, int64_t k_tok, int64_t k_head, const void *__restrict__ qw,
    const void *__restrict__ kw, int w_bf16, float w_offset, const void *__restrict__ cosp, const void *__restrict__ sinp, int R,
    const float *__restrict__ q_rstd, const float *__restrict__ k_rstd, int T, int Hq, int Hkv,
    bf16_t *__restrict__ dq_in, int64_t dq_tok, int64_t dq_head, bf16_t *__restrict__ dk_in, int64_t dk_tok,
    int64_t dk_head, float *__restrict__ part) {
    constexpr int LPR = D / 8, RPW = 64 / LPR;
    __shared__ float red[4][2][D];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int sub = lane / LPR, d0 = (lane % LPR) * 8;
    const int half_lanes = R / 16;
    const bool low = d0 < R / 2, rot = d0 < R;
    f32x8 wq, wk, aq, ak;
#pragma unroll
    for (int i = 0; i < 8; ++i) { wq[i] = norm_weight(qw, w_bf16, d0 + i) + w_offset; wk[i] = norm_weight(kw, w_bf16, d0 + i) + w_offset; aq[i] = 0.f; ak[i] = 0.f; }
    for (int64_t t = (int64_t)blockIdx.x * 4 + wv; t < T; t += (int64_t)gridDim.x * 4) {
        f32x8 c, s;
        load_cs<CS_F32>(cosp, t, R, d0, c, 1.f);
        load_cs<CS_F32>(sinp, t, R, d0, s, 0.f);
        const int H = Hq + Hkv;
        for (int r0 = 0; r0 < H; r0 += RPW) {
            const int r = r0 + sub;
            const bool live = r < H, isq = r < Hq;
            const int hh = live ? (isq ? r : r - Hq) : 0;
            const bf16_t *src = isq ? q_in + t * q_tok + hh * q_head : k_in + t * k_tok + hh * k_head;
            const bf16_t *gsrc = isq ? gq + ((int64_t)t * Hq + hh) * D : gk + ((int64_t)t * Hkv + hh) * D;
            const u32x4 z4 = {0u, 0u, 0u, 0u};
            const f32x8 x = bf8_to_f32(live ? *reinterpret_cast<const u32x4 *>(src + d0) : z4);
            const f32x8 g = bf8_to_f32(live ? *reinterpret_cast<const u32x4 *>(gsrc + d0) : z4);
            const float rstd = live ? (isq ? q_rstd + (int64_t)t * Hq : k_rstd + (int64_t)t * Hkv)[hh] : 0.f;
            const f32x8 w = isq ? wq : wk;
            f32x8 dn, xh;
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // transpose of rotate_half: dn[i] = g[i] cos[i] + (i < R/2 ? g[i+R/2] sin[i+R/2] : -g[i-R/2] sin[i-R/2])
                const float gs = g[i] * s[i];
                const float other = __shfl(gs, low ? lane + half_lanes : lane - half_lanes, 64);
                dn[i] = rot ? g[i] * c[i] + (low ? other : -other) : g[i];
                xh[i] = x[i] * rstd;
                dot += dn[i] * w[i] * xh[i];
            }
            const float mean = row_sum<LPR>(dot) * (1.f / D);
            f32x8 dx;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                dx[i] = rstd * (dn[i] * w[i] - xh[i] * mean);
                if (isq) aq[i] += dn[i] * xh[i]; else ak[i] += dn[i] * xh[i];          // dead rows carry zeros
            }
            if (live) {
                bf16_t *dst = isq ? dq_in + t * dq_tok + hh * dq_head : dk_in + t * dk_tok + hh * dk_head;
                *reinterpret_cast<u32x4 *>(dst + d0) = f32_to_bf8(dx);
            }
        }
    }
    // rows of one wave -> one value per d; then the four waves; fixed order throughout
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int m = LPR; m < 64; m <<= 1) { aq[i] += __shfl_xor(aq[i], m, 64); ak[i] += __shfl_xor(ak[i], m, 64); }
    }
    if (sub == 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { red[wv][0][d0 + i] = aq[i]; red[wv][1][d0 + i] = ak[i]; }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * D; i += 256) {
        const int which = i / D, d = i % D;
        part[((int64_t)blockIdx.x * 2 + which) * D + d] = red[0][which][d] + red[1][which][d] + red[2][which][d] + red[3][which][d];
    }
}

// dw[which][d] = sum over the workgroups' partial sums.  A workgroup of 64 x 16 threads owns 64
// consecutive d of one weight: thread (x, y) adds the partials of blocks y, y+16, ... (coalesced over x),
// then the 16 sub-sums are added in y order - the same order on every run.
__global__ __launch_bounds__(1024) void dsa_norm_weight_reduce_kernel(const float *__restrict__ part, int nblocks, int D,
                                                                      float *__restrict__ dqw, float *__restrict__ dkw) {
    __shared__ float red[16][64];
    const int x = threadIdx.x & 63, y = threadIdx.x >> 6;
    const int which = (blockIdx.x * 64) / D, d = (blockIdx.x * 64) % D + x;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;        // four loads in flight; the order of additions stays fixed
    int b = y;
    for (; b + 48 < nblocks; b += 64) {
        a0 += part[((int64_t)b * 2 + which) * D + d];
        a1 += part[((int64_t)(b + 16) * 2 + which) * D + d];
        a2 += part[((int64_t)(b + 32) * 2 + which) * D + d];
        a3 += part[((int64_t)(b + 48) * 2 + which) * D + d];
    }
    for (; b < nblocks; b += 16) a0 += part[((int64_t)b * 2 + which) * D + d];
    red[y][x] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (y == 0) {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) t += red[i][x];
        (which ? dkw : dqw)[d] = t;
    }
}

// ---- out * sigmoid(gate) (models/qwen3_5/model.py:135); rows of `width` elements, gate rows strided ----
__global__ __launch_bounds__(256) void dsa_sigmoid_gate_fwd_kernel(const bf16_t *__restrict__ x, const bf16_t *__restrict__ gate,
                                                                   int64_t gate_tok, int64_t gate_head, int D, int H, int64_t rows,
                                                                   bf16_t *__restrict__ y) {
    // one 16-byte chunk per thread and step; chunk c covers elements [8c, 8c+8) of the (rows, H*D) matrix
    const int64_t chunks = rows * H * D / 8;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += (int64_t)gridDim.x * 256) {
        const int64_t e = c * 8, t = e / ((int64_t)H * D);
        const int rem = (int)(e - t * H * D), hh = rem / D, d = rem % D;
        const f32x8 a = bf8_to_f32(*reinterpret_cast<const u32x4 *>(x + e));
        const f32x8 g = bf8_to_f32(*reinterpret_cast<const u32x4 *>(gate + t * gate_tok + hh * gate_head + d));
        f32x8 r;
#pragma unroll
        for (int i = 0; i < 8; ++i) r[i] = a[i] * bf16_round(1.f / (1.f + __expf(-g[i])));   // torch.sigmoid returns bf16
        *reinterpret_cast<u32x4 *>(y + e) = f32_to_bf8(r);
    }
}
__global__ __launch_bounds__(256) void dsa_sigmoid_gate_bwd_kernel(const bf16_t *__restrict__ gy, const bf16_t *__restrict__ x,
                                                                   const bf16_t *__restrict__ gate, int64_t gate_tok,
                                                                   int64_t gate_head, int D, int H, int64_t rows,
                                                                   bf16_t *__restrict__ dx, bf16_t *__restrict__ dgate,
                                                                   int64_t dgate_tok, int64_t dgate_head) {
    const int64_t chunks = rows * H * D / 8;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += (int64_t)gridDim.x * 256) {
        const int64_t e = c * 8, t = e / ((int64_t)H * D);
        const int rem = (int)(e - t * H * D), hh = rem / D, d = rem % D;
        const f32x8 gyv = bf8_to_f32(*reinterpret_cast<const u32x4 *>(gy + e));
        const f32x8 a = bf8_to_f32(*reinterpret_cast<const u32x4 *>(x + e));
        const f32x8 g = bf8_to_f32(*reinterpret_cast<const u32x4 *>(gate + t * gate_tok + hh * gate_head + d));
        f32x8 r1, r2;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float sg = 1.f / (1.f + __expf(-g[i]));
            r1[i] = gyv[i] * sg;
            r2[i] = gyv[i] * a[i] * sg * (1.f - sg);
        }
        *reinterpret_cast<u32x4 *>(dx + e) = f32_to_bf8(r1);
        *reinterpret_cast<u32x4 *>(dgate + t * dgate_tok + hh * dgate_head + d) = f32_to_bf8(r2);
    }
}

// ---- launchers -------------------------------------------------------------------------------------
static inline int prologue_blocks(int T) {
    const int want = (T + 3) / 4;
    return want < 1 ? 1 : (want > 2048 ? 2048 : want);
}
extern "C" int dsa_prologue_bwd_blocks(int T) { return prologue_blocks(T); }

#define PROLOGUE_SWITCH(KERNEL, ...)                                                        \
    switch (D) {                                                                            \
        case 64: if (cs_f32) hipLaunchKernelGGL((KERNEL<64, true>), __VA_ARGS__); else hipLaunchKernelGGL((KERNEL<64, false>), __VA_ARGS__); break;    \
        case 128: if (cs_f32) hipLaunchKernelGGL((KERNEL<128, true>), __VA_ARGS__); else hipLaunchKernelGGL((KERNEL<128, false>), __VA_ARGS__); break; \
        case 256: if (cs_f32) hipLaunchKernelGGL((KERNEL<256, true>), __VA_ARGS__); else hipLaunchKernelGGL((KERNEL<256, false>), __VA_ARGS__); break; \
        default: return hipErrorInvalidValue;                                               \
    }

extern "C" hipError_t dsa_launch_qk_norm_rope_fwd(const void *q_in, int64_t q_tok, int64_t q_head, const void *k_in,
                                                  int64_t k_tok, int64_t k_head, const void *qw, const void *kw, int w_bf16, float eps,
                                                  float w_offset, const void *cosp, const void *sinp, int cs_f32, int R, int T,
                                                  int Hq, int Hkv, int D, void *q_out, void *k_out, float *q_rstd,
                                                  float *k_rstd, hipStream_t stream) {
    if (T == 0) return hipSuccess;
    PROLOGUE_SWITCH(dsa_qk_norm_rope_fwd_kernel, dim3(prologue_blocks(T)), dim3(256), 0, stream, (const bf16_t *)q_in, q_tok,
                    q_head, (const bf16_t *)k_in, k_tok, k_head, qw, kw, w_bf16, eps, w_offset, cosp, sinp, R, T, Hq, Hkv,
                    (bf16_t *)q_out, (bf16_t *)k_out, q_rstd, k_rstd)
    return hipGetLastError();
}

extern "C" hipError_t dsa_launch_qk_norm_rope_bwd(const void *gq, const void *gk, const void *q_in, int64_t q_tok,
                                                  int64_t q_head, const void *k_in, int64_t k_tok, int64_t k_head,
                                                  const void *qw, const void *kw, int w_bf16, float w_offset, const void *cosp,
                                                  const void *sinp, int cs_f32, int R, const float *q_rstd,
                                                  const float *k_rstd, int T, int Hq, int Hkv, int D, void *dq_in,
                                                  int64_t dq_tok, int64_t dq_head, void *dk_in, int64_t dk_tok,
                                                  int64_t dk_head, float *dqw, float *dkw, float *part, hipStream_t stream) {
    const int nb = prologue_blocks(T);
    if (T > 0) {
        PROLOGUE_SWITCH(dsa_qk_norm_rope_bwd_kernel, dim3(nb), dim3(256), 0, stream, (const bf16_t *)gq, (const bf16_t *)gk,
                        (const bf16_t *)q_in, q_tok, q_head, (const bf16_t *)k_in, k_tok, k_head, qw, kw, w_bf16, w_offset, cosp, sinp,
                        R, q_rstd, k_rstd, T, Hq, Hkv, (bf16_t *)dq_in, dq_tok, dq_head, (bf16_t *)dk_in, dk_tok, dk_head, part)
    }
    hipLaunchKernelGGL(dsa_norm_weight_reduce_kernel, dim3(2 * D / 64), dim3(1024), 0, stream, part, T > 0 ? nb : 0, D, dqw,
                       dkw);
    return hipGetLastError();
}

extern "C" hipError_t dsa_launch_sigmoid_gate_fwd(const void *x, const void *gate, int64_t gate_tok, int64_t gate_head, int D,
                                                  int H, int64_t rows, void *y, hipStream_t stream) {
    const int64_t chunks = rows * H * D / 8;
    if (chunks == 0) return hipSuccess;
    const int nb = (int)((chunks + 255) / 256 > 16384 ? 16384 : (chunks + 255) / 256);
    hipLaunchKernelGGL(dsa_sigmoid_gate_fwd_kernel, dim3(nb), dim3(256), 0, stream, (const bf16_t *)x, (const bf16_t *)gate,
                       gate_tok, gate_head, D, H, rows, (bf16_t *)y);
    return hipGetLastError();
}
extern "C" hipError_t dsa_launch_sigmoid_gate_bwd(const void *gy, const void *x, const void *gate, int64_t gate_tok,
                                                  int64_t gate_head, int D, int H, int64_t rows, void *dx, void *dgate,
                                                  int64_t dgate_tok, int64_t dgate_head, hipStream_t stream) {
    const int64_t chunks = rows * H * D / 8;
    if (chunks == 0) return hipSuccess;
    const int nb = (int)((chunks + 255) / 256 > 16384 ? 16384 : (chunks + 255) / 256);
    hipLaunchKernelGGL(dsa_sigmoid_gate_bwd_kernel, dim3(nb), dim3(256), 0, stream, (const bf16_t *)gy, (const bf16_t *)x,
                       (const bf16_t *)gate, gate_tok, gate_head, D, H, rows, (bf16_t *)dx, (bf16_t *)dgate, dgate_tok,
                       dgate_head);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// fp32 operands on the bf16 kernels: x = hi + lo with hi = bf16(x), lo = bf16(x - hi), the parts stacked along
// head_dim into rows of 4*D bf16 so that the products of the stacked operands give back near-fp32 logits:
//   order 0: [hi, lo, hi, 0]  (q, v)        order 1: [hi, hi, lo, 0]  (k, dO)
// and the way back, out[r, :] = y[r, 0:D] + y[r, part*D:(part+1)*D] in fp32.  One thread per 4 elements.
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ void split_stack4(const float *__restrict__ x, int64_t i, int D, int order, bf16_t *__restrict__ y) {
    const int64_t r = i / (D / 4);
    const int c = (int)(i % (D / 4)) * 4;
    const f32x4 v = *reinterpret_cast<const f32x4 *>(x + r * D + c);
    const uint32_t h0 = pack2bf(v[0], v[1]), h1 = pack2bf(v[2], v[3]);
    const uint32_t l0 = pack2bf(v[0] - __uint_as_float(h0 << 16), v[1] - __uint_as_float(h0 & 0xffff0000u));
    const uint32_t l1 = pack2bf(v[2] - __uint_as_float(h1 << 16), v[3] - __uint_as_float(h1 & 0xffff0000u));
    bf16_t *o = y + r * 4 * D + c;
    const u32x2 hi = {h0, h1}, lo = {l0, l1}, z = {0u, 0u};
    *reinterpret_cast<u32x2 *>(o) = hi;
    *reinterpret_cast<u32x2 *>(o + D) = order ? hi : lo;
    *reinterpret_cast<u32x2 *>(o + 2 * D) = order ? lo : hi;
    *reinterpret_cast<u32x2 *>(o + 3 * D) = z;
}
__device__ __forceinline__ void split_combine4(const bf16_t *__restrict__ y, int64_t i, int D, int part, float *__restrict__ out) {
    const int64_t r = i / (D / 4);
    const int c = (int)(i % (D / 4)) * 4;
    const u32x2 a = *reinterpret_cast<const u32x2 *>(y + r * 4 * D + c);
    const u32x2 b = *reinterpret_cast<const u32x2 *>(y + r * 4 * D + part * D + c);
    const f32x4 o = {__uint_as_float(a[0] << 16) + __uint_as_float(b[0] << 16),
                     __uint_as_float(a[0] & 0xffff0000u) + __uint_as_float(b[0] & 0xffff0000u),
                     __uint_as_float(a[1] << 16) + __uint_as_float(b[1] << 16),
                     __uint_as_float(a[1] & 0xffff0000u) + __uint_as_float(b[1] & 0xffff0000u)};
    *reinterpret_cast<f32x4 *>(out + r * D + c) = o;
}
__global__ __launch_bounds__(256) void dsa_split_stack_kernel(const float *__restrict__ x, int64_t rows, int D, int order,
                                                               bf16_t *__restrict__ y) {
    const int64_t n4 = rows * (D / 4);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) split_stack4(x, i, D, order, y);
}
__global__ __launch_bounds__(256) void dsa_split_combine_kernel(const bf16_t *__restrict__ y, int64_t rows, int D, int part,
                                                                 float *__restrict__ out) {
    const int64_t n4 = rows * (D / 4);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) split_combine4(y, i, D, part, out);
}
// the three operands of one attention call in one launch: q-shaped (rows_q) first, then the two kv-shaped ones
__global__ __launch_bounds__(256) void dsa_split_stack_qkv_kernel(const float *__restrict__ q, const float *__restrict__ k,
                                                                   const float *__restrict__ v, int64_t rows_q, int64_t rows_kv,
                                                                   int D, bf16_t *__restrict__ yq, bf16_t *__restrict__ yk,
                                                                   bf16_t *__restrict__ yv) {
    const int64_t nq = rows_q * (D / 4), nkv = rows_kv * (D / 4);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nq + 2 * nkv; i += (int64_t)gridDim.x * 256) {
        if (i < nq) split_stack4(q, i, D, 0, yq);
        else if (i < nq + nkv) split_stack4(k, i - nq, D, 1, yk);
        else split_stack4(v, i - nq - nkv, D, 0, yv);
    }
}
__global__ __launch_bounds__(256) void dsa_split_combine_qkv_kernel(const bf16_t *__restrict__ yq, const bf16_t *__restrict__ yk,
                                                                     const bf16_t *__restrict__ yv, int64_t rows_q,
                                                                     int64_t rows_kv, int D, float *__restrict__ dq,
                                                                     float *__restrict__ dk, float *__restrict__ dv) {
    const int64_t nq = rows_q * (D / 4), nkv = rows_kv * (D / 4);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nq + 2 * nkv; i += (int64_t)gridDim.x * 256) {
        if (i < nq) split_combine4(yq, i, D, 2, dq);
        else if (i < nq + nkv) split_combine4(yk, i - nq, D, 1, dk);
        else split_combine4(yv, i - nq - nkv, D, 2, dv);
    }
}
extern "C" hipError_t dsa_launch_split_stack(const float *x, int64_t rows, int D, int order, void *y, hipStream_t stream) {
    const int64_t n4 = rows * (D / 4);
    if (n4 == 0) return hipSuccess;
    const int nb = (int)((n4 + 255) / 256 > 8192 ? 8192 : (n4 + 255) / 256);
    hipLaunchKernelGGL(dsa_split_stack_kernel, dim3(nb), dim3(256), 0, stream, x, rows, D, order, (bf16_t *)y);
    return hipGetLastError();
}
extern "C" hipError_t dsa_launch_split_combine(const void *y, int64_t rows, int D, int part, float *out, hipStream_t stream) {
    const int64_t n4 = rows * (D / 4);
    if (n4 == 0) return hipSuccess;
    const int nb = (int)((n4 + 255) / 256 > 8192 ? 8192 : (n4 + 255) / 256);
    hipLaunchKernelGGL(dsa_split_combine_kernel, dim3(nb), dim3(256), 0, stream, (const bf16_t *)y, rows, D, part, out);
    return hipGetLastError();
}
extern "C" hipError_t dsa_launch_split_stack_qkv(const float *q, const float *k, const float *v, int64_t rows_q, int64_t rows_kv,
                                                 int D, void *yq, void *yk, void *yv, hipStream_t stream) {
    const int64_t n4 = (rows_q + 2 * rows_kv) * (D / 4);
    if (n4 == 0) return hipSuccess;
    const int nb = (int)((n4 + 255) / 256 > 8192 ? 8192 : (n4 + 255) / 256);
    hipLaunchKernelGGL(dsa_split_stack_qkv_kernel, dim3(nb), dim3(256), 0, stream, q, k, v, rows_q, rows_kv, D, (bf16_t *)yq,
                       (bf16_t *)yk, (bf16_t *)yv);
    return hipGetLastError();
}
extern "C" hipError_t dsa_launch_split_combine_qkv(const void *yq, const void *yk, const void *yv, int64_t rows_q, int64_t rows_kv,
                                                   int D, float *dq, float *dk, float *dv, hipStream_t stream) {
    const int64_t n4 = (rows_q + 2 * rows_kv) * (D / 4);
    if (n4 == 0) return hipSuccess;
    const int nb = (int)((n4 + 255) / 256 > 8192 ? 8192 : (n4 + 255) / 256);
    hipLaunchKernelGGL(dsa_split_combine_qkv_kernel, dim3(nb), dim3(256), 0, stream, (const bf16_t *)yq, (const bf16_t *)yk,
                       (const bf16_t *)yv, rows_q, rows_kv, D, dq, dk, dv);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// fp32 -> bf16 (round to nearest even, the hardware conversion) of three arrays in one launch: the indexer's inputs of
// an fp32 caller.  Four elements per thread; the last one to three of an array go one by one.
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ void round4_bf16(const float *__restrict__ x, int64_t i4, int64_t n, bf16_t *__restrict__ y) {
    const int64_t i = i4 * 4;
    if (i + 4 <= n) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(x + i);
        const u32x2 o = {pack2bf(v[0], v[1]), pack2bf(v[2], v[3])};
        *reinterpret_cast<u32x2 *>(y + i) = o;
    } else {
        for (int64_t j = i; j < n; ++j) y[j] = (bf16_t)x[j];
    }
}
__global__ __launch_bounds__(256) void dsa_round_bf16_x3_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                                 const float *__restrict__ c, int64_t na, int64_t nb, int64_t nc,
                                                                 bf16_t *__restrict__ ya, bf16_t *__restrict__ yb,
                                                                 bf16_t *__restrict__ yc) {
    const int64_t qa = (na + 3) / 4, qb = (nb + 3) / 4, qc = (nc + 3) / 4;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < qa + qb + qc; i += (int64_t)gridDim.x * 256) {
        if (i < qa) round4_bf16(a, i, na, ya);
        else if (i < qa + qb) round4_bf16(b, i - qa, nb, yb);
        else round4_bf16(c, i - qa - qb, nc, yc);
    }
}
extern "C" hipError_t dsa_launch_round_bf16_x3(const float *a, const float *b, const float *c, int64_t na, int64_t nb, int64_t nc,
                                               void *ya, void *yb, void *yc, hipStream_t stream) {
    const int64_t n4 = (na + 3) / 4 + (nb + 3) / 4 + (nc + 3) / 4;
    if (n4 == 0) return hipSuccess;
    const int nb_ = (int)((n4 + 255) / 256 > 8192 ? 8192 : (n4 + 255) / 256);
    hipLaunchKernelGGL(dsa_round_bf16_x3_kernel, dim3(nb_), dim3(256), 0, stream, a, b, c, na, nb, nc, (bf16_t *)ya, (bf16_t *)yb,
                       (bf16_t *)yc);
    return hipGetLastError();
}
