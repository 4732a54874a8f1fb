// Generic NA1D kernels: any head_dim that is a multiple of 8, any window up to 80,
// any T.  They read neighbour rows straight from global memory (the cache
// hierarchy supplies the reuse) and favour simplicity; the MFMA kernels in
// na1d_mfma.hip take over for the shapes they cover.  These stay as the fallback
// and as an independent second implementation for cross-checks.
#include "na1d_common.h"

namespace na1d {
namespace generic {

constexpr int kThreads = 256;

__host__ inline unsigned grid_for(int64_t items, int per_block) {
    int64_t n = (items + per_block - 1) / per_block;
    const int64_t cap = 1 << 20;
    return (unsigned)(n < 1 ? 1 : (n > cap ? cap : n));
}

template <class DT>
__device__ inline float dot_rows(const Chunk8 *__restrict__ a, const Chunk8 *__restrict__ b, int C8) {
    float s = 0.f;
    for (int c = 0; c < C8; ++c) {
        float fa[8], fb[8];
        unpack8<DT>(a[c], fa);
        unpack8<DT>(b[c], fb);
#pragma unroll
        for (int i = 0; i < 8; ++i) s = __builtin_fmaf(fa[i], fb[i], s);
    }
    return s;
}

// ---------------------------------------------------------------- P1
// One thread per score: attn[row, j] = a[row] . b[row - L + j]   (0 if the key row is outside [0,T)).
template <class DT>
__global__ void __launch_bounds__(kThreads)
qk_kernel(float *__restrict__ attn, const Chunk8 *__restrict__ a, const Chunk8 *__restrict__ b,
          int64_t total, int64_t T, int C8, int W, int L) {
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < total; idx += stride) {
        const int64_t row = idx / W;
        const int j = (int)(idx - row * W);
        const int64_t t = row % T;
        const int64_t u = t - L + j;
        float s = 0.f;
        if (u >= 0 && u < T) s = dot_rows<DT>(a + row * C8, b + (row - L + j) * C8, C8);
        attn[idx] = s;
    }
}

// ---------------------------------------------------------------- P2
// One thread per 8 output channels: out[row, c8] = sum_j attn[row, j] * v[row - L + j, c8].
template <class DT>
__global__ void __launch_bounds__(kThreads)
av_kernel(Chunk8 *__restrict__ out, const float *__restrict__ attn, const Chunk8 *__restrict__ v,
          int64_t total, int64_t T, int C8, int W, int L) {
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < total; idx += stride) {
        const int64_t row = idx / C8;
        const int c = (int)(idx - row * C8);
        const int64_t t = row % T;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const int jlo = (int)(t < L ? L - t : 0);
        const int jhi = (int)((T - t + L) < W ? (T - t + L) : W);   // key = t-L+j < T
        for (int j = jlo; j < jhi; ++j) {
            const float p = attn[row * W + j];
            float f[8];
            unpack8<DT>(v[(row - L + j) * C8 + c], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(p, f[i], acc[i]);
        }
        out[idx] = pack8<DT>(acc);
    }
}

// ---------------------------------------------------------------- P3
// One thread per 8 output channels of a key row u:
//   out[u, c8] = sum_j attn[u + L - j, j] * x[u + L - j, c8]   over query rows inside [0,T).
template <class DT>
__global__ void __launch_bounds__(kThreads)
gather_kernel(Chunk8 *__restrict__ out, const float *__restrict__ attn, const Chunk8 *__restrict__ x,
              int64_t total, int64_t T, int C8, int W, int L) {
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < total; idx += stride) {
        const int64_t row = idx / C8;
        const int c = (int)(idx - row * C8);
        const int64_t u = row % T;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        // query t = u + L - j must satisfy 0 <= t < T
        const int jlo = (int)((u + L - (T - 1)) > 0 ? (u + L - (T - 1)) : 0);
        const int jhi = (int)((u + L + 1) < W ? (u + L + 1) : W);
        for (int j = jlo; j < jhi; ++j) {
            const int64_t r = row + L - j;
            const float s = attn[r * W + j];
            float f[8];
            unpack8<DT>(x[r * C8 + c], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(s, f[i], acc[i]);
        }
        out[idx] = pack8<DT>(acc);
    }
}

// ---------------------------------------------------------------- fused forward
// A block owns R consecutive rows of the flattened [B*T] index space.
//   phase 1: one thread per (row, j) -> logit into LDS
//   phase 2: one thread per row      -> softmax in place, log-sum-exp out
//   phase 3: one thread per (row, 8 channels) -> out
constexpr int kFwdRows = 64;

__device__ inline float logit_of(float s, float scale, const float *rpb_h, int j, bool masked) {
    float z = s * scale;
    if (rpb_h) z += rpb_h[j];
    if (masked) z += kMaskValue;
    return z;
}

template <class DT>
__global__ void __launch_bounds__(kThreads)
fused_fwd_kernel(Chunk8 *__restrict__ out, float *__restrict__ lse, const Chunk8 *__restrict__ q,
                 const Chunk8 *__restrict__ k, const Chunk8 *__restrict__ v, const float *__restrict__ rpb,
                 const int32_t *__restrict__ t_valid, int64_t rows, int64_t T, int C8, int W, int L, int H,
                 float scale, Dropout drop) {
    extern __shared__ float z[];   // [kFwdRows][W]
    const int64_t r0 = (int64_t)blockIdx.x * kFwdRows;
    const int nr = (int)((rows - r0) < kFwdRows ? (rows - r0) : kFwdRows);

    for (int idx = threadIdx.x; idx < nr * W; idx += kThreads) {
        const int r = idx / W, j = idx - r * W;
        const int64_t row = r0 + r;
        const int64_t b = row / T, t = row - b * T;
        const int64_t u = t - L + j;
        int64_t tv = T;
        if (t_valid) {
            tv = t_valid[b / H];
            tv = tv < 0 ? 0 : (tv > T ? T : tv);
        }
        float s = 0.f;
        if (u >= 0 && u < T) s = dot_rows<DT>(q + row * C8, k + (row - L + j) * C8, C8);
        z[idx] = logit_of(s, scale, rpb ? rpb + (b % H) * W : nullptr, j, t >= tv || u < 0 || u >= tv);
    }
    __syncthreads();

    if ((int)threadIdx.x < nr) {
        float *zr = z + threadIdx.x * W;
        float m = zr[0];
        for (int j = 1; j < W; ++j) m = fmaxf(m, zr[j]);
        float sum = 0.f;
        for (int j = 0; j < W; ++j) {
            const float e = fast_exp(zr[j] - m);
            zr[j] = e;
            sum += e;
        }
        const float inv = 1.0f / sum;
        for (int j = 0; j < W; ++j) zr[j] *= inv;
        if (lse) lse[r0 + threadIdx.x] = m + __logf(sum);          // of the softmax before any probability is dropped
        if (drop.threshold) {                                          // the keep rule of na1d_common.h, slot by slot
            const int64_t row = r0 + threadIdx.x, b = row / T;
            const uint32_t key = dropout_row_key(dropout_row(drop, (uint64_t)b, (int)T, (int)(row - b * T)), drop);
            for (int j = 0; j < W; ++j) zr[j] = dropout_keeps(key, j, drop) ? zr[j] * drop.inv_keep : 0.f;
        }
    }
    __syncthreads();

    for (int idx = threadIdx.x; idx < nr * C8; idx += kThreads) {
        const int r = idx / C8, c = idx - r * C8;
        const int64_t row = r0 + r;
        const int64_t t = row % T;
        const float *pr = z + r * W;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const int jlo = (int)(t < L ? L - t : 0);
        const int jhi = (int)((T - t + L) < W ? (T - t + L) : W);
        for (int j = jlo; j < jhi; ++j) {
            float f[8];
            unpack8<DT>(v[(row - L + j) * C8 + c], f);
            const float p = pr[j];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(p, f[i], acc[i]);
        }
        out[row * C8 + c] = pack8<DT>(acc);
    }
}

// ---------------------------------------------------------------- fused backward
// A block owns R consecutive rows [u0, u0+R) of ONE (batch, head) sequence, both as
// query rows (dQ, drpb) and as key rows (dK, dV).  The keys need P and dS of the
// query rows u0-Rw .. u0+R-1+L (Rw = W-1-L), so those E = R+W-1 rows are recomputed
// here and kept in LDS; nothing is accumulated across blocks except drpb.
template <class DT>
__global__ void __launch_bounds__(kThreads)
fused_bwd_kernel(Chunk8 *__restrict__ dq, Chunk8 *__restrict__ dk, Chunk8 *__restrict__ dv,
                 float *__restrict__ drpb, const Chunk8 *__restrict__ q, const Chunk8 *__restrict__ k,
                 const Chunk8 *__restrict__ v, const Chunk8 *__restrict__ o, const Chunk8 *__restrict__ go,
                 const float *__restrict__ lse, const float *__restrict__ rpb,
                 const int32_t *__restrict__ t_valid, int64_t T, int tiles, int R, int C8, int W, int L, int H,
                 float scale, Dropout drop) {
    extern __shared__ float smem[];
    const int Rw = W - 1 - L;
    const int E = R + W - 1;
    float *P = smem;               // [E][W]
    float *dS = smem + E * W;      // [E][W]
    float *delta = dS + E * W;     // [E]

    const int64_t b = blockIdx.x / tiles;
    const int64_t u0 = (int64_t)(blockIdx.x - b * tiles) * R;
    const int64_t base = b * T;    // first row of this sequence
    const int64_t e0 = u0 - Rw;    // query row of extended index 0
    int64_t tv = T;
    if (t_valid) {
        tv = t_valid[b / H];
        tv = tv < 0 ? 0 : (tv > T ? T : tv);
    }
    const float *rpb_h = rpb ? rpb + (b % H) * W : nullptr;

    for (int e = threadIdx.x; e < E; e += kThreads) {
        const int64_t t = e0 + e;
        delta[e] = (t >= 0 && t < T) ? dot_rows<DT>(go + (base + t) * C8, o + (base + t) * C8, C8) : 0.f;
    }
    __syncthreads();

    for (int idx = threadIdx.x; idx < E * W; idx += kThreads) {
        const int e = idx / W, j = idx - e * W;
        const int64_t t = e0 + e;
        float p = 0.f, ds = 0.f;
        if (t >= 0 && t < T) {
            const int64_t u = t - L + j;
            float s = 0.f, dp = 0.f;
            if (u >= 0 && u < T) {
                s = dot_rows<DT>(q + (base + t) * C8, k + (base + u) * C8, C8);
                dp = dot_rows<DT>(go + (base + t) * C8, v + (base + u) * C8, C8);
            }
            const float zz = logit_of(s, scale, rpb_h, j, t >= tv || u < 0 || u >= tv);
            p = fast_exp(zz - lse[base + t]);
            if (drop.threshold) {      // O = (D * P) V with D = 0 or 1 / (1 - p_drop): dP carries D, and so does the P that dV sees
                const uint32_t key = dropout_row_key(dropout_row(drop, (uint64_t)b, (int)T, (int)t), drop);
                const float f = dropout_keeps(key, j, drop) ? drop.inv_keep : 0.f;
                dp *= f;
                ds = p * (dp - delta[e]);      // delta = rowsum(dO * O) is that of the dropped output already
                p *= f;
            } else {
                ds = p * (dp - delta[e]);
            }
        }
        P[idx] = p;
        dS[idx] = ds;
    }
    __syncthreads();

    const int nr = (int)((T - u0) < R ? (T - u0) : R);
    for (int idx = threadIdx.x; idx < nr * C8; idx += kThreads) {
        const int r = idx / C8, c = idx - r * C8;
        const int64_t u = u0 + r;
        float aq[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float ak[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float av_[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < W; ++j) {
            // dQ[u] += dS[u, j] * k[u - L + j]
            const int64_t key = u - L + j;
            if (key >= 0 && key < T) {
                float f[8];
                unpack8<DT>(k[(base + key) * C8 + c], f);
                const float g = dS[(r + Rw) * W + j];
#pragma unroll
                for (int i = 0; i < 8; ++i) aq[i] = __builtin_fmaf(g, f[i], aq[i]);
            }
            // dK[u] += dS[t, j] * q[t],  dV[u] += P[t, j] * dO[t],  t = u + L - j
            const int64_t t = u + L - j;
            if (t >= 0 && t < T) {
                const int e = r + L - j + Rw;
                const float g = dS[e * W + j], pp = P[e * W + j];
                float fq[8], fo[8];
                unpack8<DT>(q[(base + t) * C8 + c], fq);
                unpack8<DT>(go[(base + t) * C8 + c], fo);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    ak[i] = __builtin_fmaf(g, fq[i], ak[i]);
                    av_[i] = __builtin_fmaf(pp, fo[i], av_[i]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            aq[i] *= scale;
            ak[i] *= scale;
        }
        dq[(base + u) * C8 + c] = pack8<DT>(aq);
        dk[(base + u) * C8 + c] = pack8<DT>(ak);
        dv[(base + u) * C8 + c] = pack8<DT>(av_);
    }

    if (drpb && (int)threadIdx.x < W) {
        const int j = threadIdx.x;
        float s = 0.f;
        for (int r = 0; r < nr; ++r) s += dS[(r + Rw) * W + j];
        atomicAdd(drpb + (b % H) * W + j, s);
    }
}

// ---------------------------------------------------------------- launchers
#define NA1D_BY_DTYPE(CALL)                       \
    if (dtype == NA1D_BF16) { using DT = BF16; CALL; } \
    else                    { using DT = FP16; CALL; }

int qk(float *attn, const void *a, const void *b, const Geom &g, int dtype, hipStream_t s) {
    const int64_t total = g.B * g.T * g.W;
    NA1D_BY_DTYPE((qk_kernel<DT><<<grid_for(total, kThreads), kThreads, 0, s>>>(
        attn, (const Chunk8 *)a, (const Chunk8 *)b, total, g.T, g.C / 8, g.W, g.L)));
    return launch_status();
}

int av(void *out, const float *attn, const void *v, const Geom &g, int dtype, hipStream_t s) {
    const int64_t total = g.B * g.T * (g.C / 8);
    NA1D_BY_DTYPE((av_kernel<DT><<<grid_for(total, kThreads), kThreads, 0, s>>>(
        (Chunk8 *)out, attn, (const Chunk8 *)v, total, g.T, g.C / 8, g.W, g.L)));
    return launch_status();
}

int gather(void *out, const float *attn, const void *x, const Geom &g, int dtype, hipStream_t s) {
    const int64_t total = g.B * g.T * (g.C / 8);
    NA1D_BY_DTYPE((gather_kernel<DT><<<grid_for(total, kThreads), kThreads, 0, s>>>(
        (Chunk8 *)out, attn, (const Chunk8 *)x, total, g.T, g.C / 8, g.W, g.L)));
    return launch_status();
}

int fused_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
              const int32_t *t_valid, const Geom &g, float scale, int dtype, hipStream_t s) {
    const int64_t rows = g.B * g.T;
    const int64_t blocks = (rows + kFwdRows - 1) / kFwdRows;
    if (blocks > 0x7fffffffLL) return NA1D_ERR_SHAPE;
    const size_t smem = (size_t)kFwdRows * g.W * sizeof(float);
    NA1D_BY_DTYPE((fused_fwd_kernel<DT><<<(unsigned)blocks, kThreads, smem, s>>>(
        (Chunk8 *)out, lse, (const Chunk8 *)q, (const Chunk8 *)k, (const Chunk8 *)v, rpb, t_valid, rows, g.T,
        g.C / 8, g.W, g.L, g.H, scale, g.drop)));
    return launch_status();
}

int fused_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
              const void *out, const void *dout, const float *lse, const float *rpb,
              const int32_t *t_valid, const Geom &g, float scale, int dtype, hipStream_t s) {
    int R = 32;
    auto bytes = [&](int r) { return (size_t)(2 * (r + g.W - 1) * g.W + (r + g.W - 1)) * sizeof(float); };
    while (R > 8 && bytes(R) > 60 * 1024) R /= 2;
    const int64_t tiles = (g.T + R - 1) / R;
    const int64_t blocks = tiles * g.B;
    if (blocks > 0x7fffffffLL) return NA1D_ERR_SHAPE;
    NA1D_BY_DTYPE((fused_bwd_kernel<DT><<<(unsigned)blocks, kThreads, bytes(R), s>>>(
        (Chunk8 *)dq, (Chunk8 *)dk, (Chunk8 *)dv, drpb, (const Chunk8 *)q, (const Chunk8 *)k, (const Chunk8 *)v,
        (const Chunk8 *)out, (const Chunk8 *)dout, lse, rpb, t_valid, g.T, (int)tiles, R, g.C / 8, g.W, g.L, g.H,
        scale, g.drop)));
    return launch_status();
}

}  // namespace generic
}  // namespace na1d
