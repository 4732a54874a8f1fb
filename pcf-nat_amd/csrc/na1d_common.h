// Shared device helpers for the NA1D kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "na1d.h"

namespace na1d {

constexpr float kMaskValue = -100.0f;   // additive mask of the reference model (models/PCF_NATransformer.py:98)
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// 16-bit element types.  Values travel as raw uint16_t; conversion is explicit.
struct BF16 {
    static constexpr int tag = NA1D_BF16;
    __device__ static inline float to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
    // round to nearest even; NaN stays NaN
    __device__ static inline uint16_t from_f32(float f) {
        uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
        u += 0x7fffu + ((u >> 16) & 1u);
        return (uint16_t)(u >> 16);
    }
};

struct FP16 {
    static constexpr int tag = NA1D_FP16;
    __device__ static inline float to_f32(uint16_t h) {
        _Float16 x;
        __builtin_memcpy(&x, &h, 2);
        return (float)x;
    }
    __device__ static inline uint16_t from_f32(float f) {
        _Float16 x = (_Float16)f;   // v_cvt_f16_f32, round to nearest even
        uint16_t h;
        __builtin_memcpy(&h, &x, 2);
        return h;
    }
};

// Eight consecutive 16-bit channels = one 128-bit access.
struct alignas(16) Chunk8 {
    uint32_t w[4];
};

template <class DT>
__device__ inline void unpack8(const Chunk8 &c, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = DT::to_f32((uint16_t)(c.w[i] & 0xffffu));
        f[2 * i + 1] = DT::to_f32((uint16_t)(c.w[i] >> 16));
    }
}

template <class DT>
__device__ inline Chunk8 pack8(const float (&f)[8]) {
    Chunk8 c;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        c.w[i] = (uint32_t)DT::from_f32(f[2 * i]) | ((uint32_t)DT::from_f32(f[2 * i + 1]) << 16);
    return c;
}

__device__ inline float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }

// Attention dropout of the fused operator.  Whether probability (b, t, j) - packed sequence b, query row t,
// window slot j - survives is a pure function of (seed, b * T + t, j), so that the forward, the backward and any
// kernel variant agree without storing a mask:
//     key  = mix32(mix32(lo32(row) ^ lo32(seed)) + hi32(row) * 0x9E3779B9 + hi32(seed)),   row = b * T + t
//     keep = mix32(key ^ (j * 0x9E3779B9)) >= threshold,                                   threshold = floor(p * 2^32)
// with mix32 the 32-bit finaliser x ^= x >> 16; x *= 0x7feb352d; x ^= x >> 15; x *= 0x846ca68b; x ^= x >> 16.
// Survivors are scaled by 1 / (1 - p).  threshold 0 switches it off.
// A launch on every d-th row of longer sequences (a dilated window's residue class) names its rows by their place in
// the whole sequence: row = b * seq_rows + row_offset + row_stride * t for row t of the launch's sequence b.
struct Dropout {
    uint32_t threshold = 0, seed_lo = 0, seed_hi = 0;
    float inv_keep = 1.f;
    uint32_t row_stride = 1, row_offset = 0, seq_rows = 0;      // seq_rows 0: the launch's own T
};
inline Dropout make_dropout(float p, uint64_t seed, uint32_t row_stride = 1, uint32_t row_offset = 0, uint32_t seq_rows = 0) {
    Dropout d;
    d.row_stride = row_stride;
    d.row_offset = row_offset;
    d.seq_rows = seq_rows;
    if (p > 0.f) {
        const double t = (double)p * 4294967296.0;
        d.threshold = t >= 4294967295.0 ? 0xffffffffu : (uint32_t)t;
        d.seed_lo = (uint32_t)seed;
        d.seed_hi = (uint32_t)(seed >> 32);
        d.inv_keep = (float)(1.0 / (1.0 - (double)p));
    }
    return d;
}
__host__ __device__ inline uint32_t mix32(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}
__host__ __device__ inline uint32_t dropout_row_key(uint64_t row, const Dropout &d) {
    return mix32(mix32((uint32_t)row ^ d.seed_lo) + (uint32_t)(row >> 32) * 0x9E3779B9u + d.seed_hi);
}
__host__ __device__ inline uint64_t dropout_row(const Dropout &d, uint64_t b, int T, int t) {
    return b * (d.seq_rows ? d.seq_rows : (uint32_t)T) + d.row_offset + (uint64_t)d.row_stride * (uint32_t)t;
}
__host__ __device__ inline bool dropout_keeps(uint32_t row_key, int slot, const Dropout &d) {
    return mix32(row_key ^ ((uint32_t)slot * 0x9E3779B9u)) >= d.threshold;
}

// Problem description shared by every launcher.
struct Geom {
    int64_t B, T;
    int C, W, L;      // head_dim, window, left
    int H;            // heads (B % H == 0); 1 for the un-fused entry points
    Dropout drop;     // fused operator only; off by default
};

// Element strides of a [samples, heads, T, C] view of a tensor whose channels are contiguous.  The packed
// [B = samples * heads, T, C] tensor of the reference is {H*T*C, T*C, C}; a head-interleaved projection
// output [N, T, 3, H, C] is {T*3*H*C, C, 3*H*C} behind a base pointer that selects q, k or v.
struct Layout {
    int64_t sample, head, row;
};
inline Layout packed_layout(const Geom &g) { return Layout{(int64_t)g.H * g.T * g.C, g.T * g.C, g.C}; }

// Optional pair of events that the fused launches of the calling thread record tightly around the kernel
// (hipExtLaunchKernel: the dispatch's own start and end, what a profiler's kernel trace reports) - see
// na1d_profile_events() in na1d.h.  Null, the default, means ordinary launches.
struct LaunchEvents {
    hipEvent_t start = nullptr, stop = nullptr;
    bool refused = false;   // a launch was asked to record them on a capturing stream: reported by launch_status()
    char kernel[96] = "";   // name of the last kernel launched with events set (na1d_profile_last_kernel)
};
LaunchEvents &launch_events();   // thread-local, lives in na1d_api.cpp

// Host-side launch status check.
inline int launch_status() {
    LaunchEvents &ev = launch_events();
    const bool refused = ev.refused;
    ev.refused = false;
    return hipGetLastError() == hipSuccess && !refused ? NA1D_OK : NA1D_ERR_LAUNCH;
}

// ---- generic (any C % 8 == 0, any W <= 80) kernels: na1d_generic.hip -------
namespace generic {
int qk(float *attn, const void *a, const void *b, const Geom &g, int dtype, hipStream_t s);
int av(void *out, const float *attn, const void *v, const Geom &g, int dtype, hipStream_t s);
int gather(void *out, const float *attn, const void *x, const Geom &g, int dtype, hipStream_t s);
int fused_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
              const int32_t *t_valid, const Geom &g, float scale, int dtype, hipStream_t s);
int fused_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
              const void *out, const void *dout, const float *lse, const float *rpb,
              const int32_t *t_valid, const Geom &g, float scale, int dtype, hipStream_t s);
}  // namespace generic

// ---- MFMA kernels for the shapes they cover: na1d_mfma.hip ------------------
// Same signatures; each returns NA1D_ERR_UNSUPPORTED when the shape is not
// covered, and the caller then falls back to the generic kernel.
namespace mfma {
int qk(float *attn, const void *a, const void *b, const Geom &g, int dtype, hipStream_t s);
int av(void *out, const float *attn, const void *v, const Geom &g, int dtype, hipStream_t s);
int gather(void *out, const float *attn, const void *x, const Geom &g, int dtype, hipStream_t s);
// `in` lays out q, k, v (and dq, dk, dv); `out` lays out out and dout.
int fused_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
              const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &out_layout, float scale,
              int dtype, hipStream_t s);
int fused_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
              const void *out, const void *dout, const float *lse, const float *rpb,
              const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &out_layout, float scale,
              int dtype, float *workspace, int64_t workspace_bytes, hipStream_t s);
int64_t fused_bwd_workspace_bytes(const Geom &g, int dtype);   // 0 when the shape is not covered
// Device address, on the current device, of the library's static scratch array (kStaticScratchBytes bytes).
constexpr int64_t kStaticScratchBytes = NA1D_NOALLOC_SCRATCH_BYTES;
int static_scratch(float **ptr);
// wide windows (W up to 80, any split of it): na1d_mfma_wide.hip
int wide_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
             const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &out_layout, float scale,
             int dtype, hipStream_t s);
int wide_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v, const void *dout,
             const float *lse, const float *rpb, const int32_t *t_valid, const Geom &g, const Layout &in,
             const Layout &out_layout, float scale, int dtype, float *workspace, int64_t workspace_bytes, hipStream_t s);
int64_t wide_bwd_workspace_bytes(const Geom &g);               // 0 when the shape is not covered
// Dense attention over whole sequences (the models' global layers); g.W and g.L are not used.
int global_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const int32_t *t_valid,
               const Geom &g, float scale, int dtype, hipStream_t s);
int global_bwd(void *dq, void *dk, void *dv, float *delta, const void *q, const void *k, const void *v, const void *out,
               const void *dout, const float *lse, const int32_t *t_valid, const Geom &g, float scale, int dtype,
               hipStream_t s);
}  // namespace mfma

}  // namespace na1d
