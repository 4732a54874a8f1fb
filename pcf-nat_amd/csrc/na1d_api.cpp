// C ABI of libna1d: argument validation and dispatch.  No torch types, no allocation; kernels go to the stream
// that is passed in.  State that outlives a call: the calling thread's profiling events, the process-wide
// kernel-family switch, and the per-GPU scratch array of na1d_fused_backward_noalloc (na1d_mfma.hip).
#include <atomic>
#include <cstdlib>

#include "na1d_common.h"

namespace na1d {
LaunchEvents &launch_events() {
    static thread_local LaunchEvents events;
    return events;
}
}  // namespace na1d

namespace {

using na1d::Geom;

inline bool misaligned(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }
// The kernels fold the bias into the scores before the scale, which takes a positive one (false for NaN too).
inline bool bad_scale(float scale) { return !(scale > 0.f && scale <= 3.0e38f); }

// Shape checks shared by every entry point.  Returns NA1D_OK, an error, or +1 for
// "nothing to do".
int check_shape(int64_t B, int64_t T, int64_t C, int64_t W, int64_t left, int64_t H, int dtype, Geom &g) {
    if (dtype != NA1D_BF16 && dtype != NA1D_FP16) return NA1D_ERR_DTYPE;
    if (C <= 0 || C % 8 != 0 || C > (1 << 20)) return NA1D_ERR_HEAD_DIM;
    if (W < 1 || W > NA1D_MAX_WINDOW || left < 0 || left >= W) return NA1D_ERR_WINDOW;
    if (B < 0 || T < 0 || H < 1 || B % H != 0) return NA1D_ERR_SHAPE;
    if (B == 0 || T == 0) return 1;
    const int64_t widest = C > W ? C : W;
    if (T > (INT64_MAX / 8) / widest || B > (INT64_MAX / 8) / (T * widest)) return NA1D_ERR_SHAPE;
    g.B = B;
    g.T = T;
    g.C = (int)C;
    g.W = (int)W;
    g.L = (int)left;
    g.H = (int)H;
    return NA1D_OK;
}

// Shape checks plus the three pointers every entry point has.
int check(const void *o, const void *a, const void *b, int64_t B, int64_t T, int64_t C, int64_t W, int64_t left,
          int64_t H, int dtype, Geom &g) {
    const int st = check_shape(B, T, C, W, left, H, dtype, g);
    if (st != NA1D_OK) return st;
    if (!o || !a || !b) return NA1D_ERR_NULL;
    if (misaligned(o) || misaligned(a) || misaligned(b)) return NA1D_ERR_ALIGN;
    return NA1D_OK;
}

// {sample, head, row} element strides of a strided entry point: multiples of 8 elements (16 bytes), rows at
// least C apart, nothing negative.
int check_layout(const int64_t *strides, const Geom &g, na1d::Layout &l) {
    if (!strides) return NA1D_ERR_NULL;
    l = na1d::Layout{strides[0], strides[1], strides[2]};
    if (l.sample < 0 || l.head < 0 || l.row < g.C) return NA1D_ERR_SHAPE;
    if (l.sample % 8 || l.head % 8 || l.row % 8) return NA1D_ERR_ALIGN;
    if (l.sample > INT64_MAX / 4 / (g.B / g.H) || l.head > INT64_MAX / 4 / g.H || l.row > INT64_MAX / 4 / g.T)
        return NA1D_ERR_SHAPE;
    return NA1D_OK;
}

#define NA1D_CHECK(...)                     \
    Geom g;                                 \
    {                                       \
        const int st = check(__VA_ARGS__);  \
        if (st != NA1D_OK) return st > 0 ? NA1D_OK : st; \
    }

// The generic kernels are a second, independent implementation that the tests cross-check the matrix-core
// kernels against.  NA1D_FORCE_GENERIC=1 in the environment when the library is first called, or
// na1d_force_generic(1) at any time, routes every call to them.
std::atomic<int> &generic_forced() {
    static std::atomic<int> flag{[] {
        const char *e = std::getenv("NA1D_FORCE_GENERIC");
        return (e && e[0] == '1') ? 1 : 0;
    }()};
    return flag;
}
inline bool mfma_allowed() { return generic_forced().load(std::memory_order_relaxed) == 0; }

// The matrix-core forward: the two/three-block kernel where it covers the window, else the wide-window one.
int mfma_fused_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
                   const int32_t *t_valid, const Geom &g, const na1d::Layout &in, const na1d::Layout &outl, float scale,
                   int dtype, hipStream_t s) {
    const int st = na1d::mfma::fused_fwd(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, dtype, s);
    if (st != NA1D_ERR_UNSUPPORTED) return st;
    return na1d::mfma::wide_fwd(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, dtype, s);
}

int mfma_fused_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
                   const void *out, const void *dout, const float *lse, const float *rpb, const int32_t *t_valid,
                   const Geom &g, const na1d::Layout &in, const na1d::Layout &outl, float scale, int dtype,
                   float *workspace, int64_t workspace_bytes, hipStream_t s) {
    const int st = na1d::mfma::fused_bwd(dq, dk, dv, drpb, q, k, v, out, dout, lse, rpb, t_valid, g, in, outl, scale,
                                         dtype, workspace, workspace_bytes, s);
    if (st != NA1D_ERR_UNSUPPORTED) return st;
    return na1d::mfma::wide_bwd(dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, g, in, outl, scale, dtype, workspace,
                                workspace_bytes, s);
}

int band_qk(void *attn, const void *a, const void *b, const Geom &g, int dtype, hipStream_t s) {
    const int st = mfma_allowed() ? na1d::mfma::qk((float *)attn, a, b, g, dtype, s) : NA1D_ERR_UNSUPPORTED;
    return st == NA1D_ERR_UNSUPPORTED ? na1d::generic::qk((float *)attn, a, b, g, dtype, s) : st;
}
int band_av(void *out, const void *attn, const void *v, const Geom &g, int dtype, hipStream_t s) {
    const int st = mfma_allowed() ? na1d::mfma::av(out, (const float *)attn, v, g, dtype, s) : NA1D_ERR_UNSUPPORTED;
    return st == NA1D_ERR_UNSUPPORTED ? na1d::generic::av(out, (const float *)attn, v, g, dtype, s) : st;
}
int band_gather(void *out, const void *attn, const void *x, const Geom &g, int dtype, hipStream_t s) {
    const int st = mfma_allowed() ? na1d::mfma::gather(out, (const float *)attn, x, g, dtype, s) : NA1D_ERR_UNSUPPORTED;
    return st == NA1D_ERR_UNSUPPORTED ? na1d::generic::gather(out, (const float *)attn, x, g, dtype, s) : st;
}

}  // namespace

extern "C" {

int na1d_version(void) { return 100; }

const char *na1d_status_string(int status) {
    switch (status) {
        case NA1D_OK: return "ok";
        case NA1D_ERR_NULL: return "a required pointer is NULL";
        case NA1D_ERR_DTYPE: return "dtype must be NA1D_BF16 (0) or NA1D_FP16 (1)";
        case NA1D_ERR_HEAD_DIM: return "head_dim must be a positive multiple of 8";
        case NA1D_ERR_WINDOW: return "need 1 <= win_size <= 80 and 0 <= left < win_size";
        case NA1D_ERR_SHAPE: return "bad B/T/H (negative, B not a multiple of H, or too large)";
        case NA1D_ERR_ALIGN: return "tensor pointers must be 16-byte aligned";
        case NA1D_ERR_LAUNCH: return "HIP rejected the kernel launch";
        case NA1D_ERR_UNSUPPORTED: return "no kernel built for these arguments";
        case NA1D_ERR_TOO_LARGE: return "the problem needs more scratch than NA1D_NOALLOC_SCRATCH_BYTES";
        case NA1D_ERR_WORKSPACE: return "the workspace is smaller than the size the *_workspace_bytes() query returns";
        case NA1D_ERR_SCALE: return "scale must be a finite number above zero";
        default: return "unknown status";
    }
}

int na1d_qk_forward(void *attn, const void *q, const void *k, int64_t B, int64_t T, int64_t C, int64_t W,
                    int64_t left, int dtype, void *stream) {
    NA1D_CHECK(attn, q, k, B, T, C, W, left, 1, dtype, g);
    return band_qk(attn, q, k, g, dtype, (hipStream_t)stream);
}

int na1d_a_backward(void *dattn, const void *dout, const void *v, int64_t B, int64_t T, int64_t C, int64_t W,
                    int64_t left, int dtype, void *stream) {
    NA1D_CHECK(dattn, dout, v, B, T, C, W, left, 1, dtype, g);
    return band_qk(dattn, dout, v, g, dtype, (hipStream_t)stream);
}

int na1d_av_forward(void *out, const void *attn, const void *v, int64_t B, int64_t T, int64_t C, int64_t W,
                    int64_t left, int dtype, void *stream) {
    NA1D_CHECK(out, attn, v, B, T, C, W, left, 1, dtype, g);
    return band_av(out, attn, v, g, dtype, (hipStream_t)stream);
}

int na1d_q_backward(void *dq, const void *dattn, const void *k, int64_t B, int64_t T, int64_t C, int64_t W,
                    int64_t left, int dtype, void *stream) {
    NA1D_CHECK(dq, dattn, k, B, T, C, W, left, 1, dtype, g);
    return band_av(dq, dattn, k, g, dtype, (hipStream_t)stream);
}

int na1d_k_backward(void *dk, const void *dattn, const void *q, int64_t B, int64_t T, int64_t C, int64_t W,
                    int64_t left, int dtype, void *stream) {
    NA1D_CHECK(dk, dattn, q, B, T, C, W, left, 1, dtype, g);
    return band_gather(dk, dattn, q, g, dtype, (hipStream_t)stream);
}

int na1d_v_backward(void *dv, const void *attn, const void *dout, int64_t B, int64_t T, int64_t C, int64_t W,
                    int64_t left, int dtype, void *stream) {
    NA1D_CHECK(dv, attn, dout, B, T, C, W, left, 1, dtype, g);
    return band_gather(dv, attn, dout, g, dtype, (hipStream_t)stream);
}

int na1d_fused_forward(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
                       const int32_t *t_valid, int64_t B, int64_t H, int64_t T, int64_t C, int64_t W,
                       int64_t left, float scale, int dtype, void *stream) {
    NA1D_CHECK(out, q, k, B, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!v) return NA1D_ERR_NULL;
    if (misaligned(v)) return NA1D_ERR_ALIGN;
    const na1d::Layout packed = na1d::packed_layout(g);
    const int st = mfma_allowed() ? mfma_fused_fwd(out, lse, q, k, v, rpb, t_valid, g, packed, packed, scale, dtype,
                                                   (hipStream_t)stream)
                                  : NA1D_ERR_UNSUPPORTED;
    if (st != NA1D_ERR_UNSUPPORTED) return st;
    return na1d::generic::fused_fwd(out, lse, q, k, v, rpb, t_valid, g, scale, dtype, (hipStream_t)stream);
}

int na1d_fused_backward(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
                        const void *out, const void *dout, const float *lse, const float *rpb,
                        const int32_t *t_valid, int64_t B, int64_t H, int64_t T, int64_t C, int64_t W,
                        int64_t left, float scale, int dtype, void *workspace, int64_t workspace_bytes,
                        void *stream) {
    NA1D_CHECK(dq, q, k, B, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!dk || !dv || !v || !out || !dout || !lse) return NA1D_ERR_NULL;
    if (misaligned(dk) || misaligned(dv) || misaligned(v) || misaligned(out) || misaligned(dout))
        return NA1D_ERR_ALIGN;
    if (workspace && misaligned(workspace)) return NA1D_ERR_ALIGN;
    const na1d::Layout packed = na1d::packed_layout(g);
    const int st = mfma_allowed() ? mfma_fused_bwd(dq, dk, dv, drpb, q, k, v, out, dout, lse, rpb, t_valid, g,
                                                   packed, packed, scale, dtype, (float *)workspace,
                                                          workspace ? workspace_bytes : 0, (hipStream_t)stream)
                                  : NA1D_ERR_UNSUPPORTED;
    if (st != NA1D_ERR_UNSUPPORTED) return st;
    return na1d::generic::fused_bwd(dq, dk, dv, drpb, q, k, v, out, dout, lse, rpb, t_valid, g, scale, dtype,
                                    (hipStream_t)stream);   // the generic kernel has no use for the workspace
}

int na1d_fused_forward_strided(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
                               const int32_t *t_valid, int64_t N, int64_t H, int64_t T, int64_t C, int64_t W,
                               int64_t left, float scale, int dtype, const int64_t *qkv_strides,
                               const int64_t *out_strides, void *stream) {
    if (N < 0 || H < 1 || N > INT64_MAX / H) return NA1D_ERR_SHAPE;
    NA1D_CHECK(out, q, k, N * H, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!v) return NA1D_ERR_NULL;
    if (misaligned(v)) return NA1D_ERR_ALIGN;
    na1d::Layout in, outl;
    const int ls = check_layout(qkv_strides, g, in), lo = check_layout(out_strides, g, outl);
    if (ls != NA1D_OK || lo != NA1D_OK) return ls != NA1D_OK ? ls : lo;
    if (!mfma_allowed()) return NA1D_ERR_UNSUPPORTED;
    return mfma_fused_fwd(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, dtype, (hipStream_t)stream);
}

int na1d_fused_backward_strided(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k,
                                const void *v, const void *dout, const float *lse, const float *rpb,
                                const int32_t *t_valid, int64_t N, int64_t H, int64_t T, int64_t C, int64_t W,
                                int64_t left, float scale, int dtype, const int64_t *qkv_strides,
                                const int64_t *out_strides, void *workspace, int64_t workspace_bytes,
                                void *stream) {
    if (N < 0 || H < 1 || N > INT64_MAX / H) return NA1D_ERR_SHAPE;
    NA1D_CHECK(dq, q, k, N * H, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!dk || !dv || !v || !dout || !lse) return NA1D_ERR_NULL;
    if (misaligned(dk) || misaligned(dv) || misaligned(v) || misaligned(dout)) return NA1D_ERR_ALIGN;
    if (workspace && misaligned(workspace)) return NA1D_ERR_ALIGN;
    na1d::Layout in, outl;
    const int ls = check_layout(qkv_strides, g, in), lo = check_layout(out_strides, g, outl);
    if (ls != NA1D_OK || lo != NA1D_OK) return ls != NA1D_OK ? ls : lo;
    if (!mfma_allowed()) return NA1D_ERR_UNSUPPORTED;
    return mfma_fused_bwd(dq, dk, dv, drpb, q, k, v, nullptr, dout, lse, rpb, t_valid, g, in, outl, scale, dtype,
                          (float *)workspace, workspace ? workspace_bytes : 0, (hipStream_t)stream);
}

int na1d_fused_forward_dropout(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
                               const int32_t *t_valid, int64_t B, int64_t H, int64_t T, int64_t C, int64_t W,
                               int64_t left, float scale, int dtype, float p_drop, uint64_t seed, void *stream) {
    NA1D_CHECK(out, q, k, B, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!v) return NA1D_ERR_NULL;
    if (misaligned(v)) return NA1D_ERR_ALIGN;
    if (!(p_drop >= 0.f && p_drop < 1.f)) return NA1D_ERR_SHAPE;
    g.drop = na1d::make_dropout(p_drop, seed);
    const na1d::Layout packed = na1d::packed_layout(g);
    const int st = mfma_allowed() ? mfma_fused_fwd(out, lse, q, k, v, rpb, t_valid, g, packed, packed, scale, dtype,
                                                   (hipStream_t)stream)
                                  : NA1D_ERR_UNSUPPORTED;
    if (st != NA1D_ERR_UNSUPPORTED) return st;
    return na1d::generic::fused_fwd(out, lse, q, k, v, rpb, t_valid, g, scale, dtype, (hipStream_t)stream);
}

int na1d_fused_backward_dropout(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
                                const void *out, const void *dout, const float *lse, const float *rpb,
                                const int32_t *t_valid, int64_t B, int64_t H, int64_t T, int64_t C, int64_t W,
                                int64_t left, float scale, int dtype, float p_drop, uint64_t seed, void *workspace,
                                int64_t workspace_bytes, void *stream) {
    NA1D_CHECK(dq, q, k, B, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!dk || !dv || !v || !out || !dout || !lse) return NA1D_ERR_NULL;
    if (misaligned(dk) || misaligned(dv) || misaligned(v) || misaligned(out) || misaligned(dout))
        return NA1D_ERR_ALIGN;
    if (workspace && misaligned(workspace)) return NA1D_ERR_ALIGN;
    if (!(p_drop >= 0.f && p_drop < 1.f)) return NA1D_ERR_SHAPE;
    g.drop = na1d::make_dropout(p_drop, seed);
    const na1d::Layout packed = na1d::packed_layout(g);
    const int st = mfma_allowed() ? mfma_fused_bwd(dq, dk, dv, drpb, q, k, v, out, dout, lse, rpb, t_valid, g,
                                                   packed, packed, scale, dtype, (float *)workspace,
                                                   workspace ? workspace_bytes : 0, (hipStream_t)stream)
                                  : NA1D_ERR_UNSUPPORTED;
    if (st != NA1D_ERR_UNSUPPORTED) return st;
    return na1d::generic::fused_bwd(dq, dk, dv, drpb, q, k, v, out, dout, lse, rpb, t_valid, g, scale, dtype,
                                    (hipStream_t)stream);
}

int na1d_fused_forward_strided_dropout(void *out, float *lse, const void *q, const void *k, const void *v,
                                       const float *rpb, const int32_t *t_valid, int64_t N, int64_t H, int64_t T,
                                       int64_t C, int64_t W, int64_t left, float scale, int dtype,
                                       const int64_t *qkv_strides, const int64_t *out_strides, float p_drop,
                                       uint64_t seed, int64_t row_stride, int64_t row_offset, int64_t seq_rows,
                                       void *stream) {
    if (N < 0 || H < 1 || N > INT64_MAX / H) return NA1D_ERR_SHAPE;
    NA1D_CHECK(out, q, k, N * H, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!v) return NA1D_ERR_NULL;
    if (misaligned(v)) return NA1D_ERR_ALIGN;
    if (!(p_drop >= 0.f && p_drop < 1.f)) return NA1D_ERR_SHAPE;
    if (row_stride < 1 || row_offset < 0 || row_offset >= row_stride || seq_rows < row_offset + row_stride * (T - 1) + 1 ||
        seq_rows > 0x7fffffffLL)
        return NA1D_ERR_SHAPE;
    g.drop = na1d::make_dropout(p_drop, seed, (uint32_t)row_stride, (uint32_t)row_offset, (uint32_t)seq_rows);
    na1d::Layout in, outl;
    const int ls = check_layout(qkv_strides, g, in), lo = check_layout(out_strides, g, outl);
    if (ls != NA1D_OK || lo != NA1D_OK) return ls != NA1D_OK ? ls : lo;
    if (!mfma_allowed()) return NA1D_ERR_UNSUPPORTED;
    return mfma_fused_fwd(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, dtype, (hipStream_t)stream);
}

int na1d_fused_backward_strided_dropout(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k,
                                        const void *v, const void *dout, const float *lse, const float *rpb,
                                        const int32_t *t_valid, int64_t N, int64_t H, int64_t T, int64_t C, int64_t W,
                                        int64_t left, float scale, int dtype, const int64_t *qkv_strides,
                                        const int64_t *out_strides, float p_drop, uint64_t seed, int64_t row_stride,
                                        int64_t row_offset, int64_t seq_rows, void *workspace, int64_t workspace_bytes,
                                        void *stream) {
    if (N < 0 || H < 1 || N > INT64_MAX / H) return NA1D_ERR_SHAPE;
    NA1D_CHECK(dq, q, k, N * H, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!dk || !dv || !v || !dout || !lse) return NA1D_ERR_NULL;
    if (misaligned(dk) || misaligned(dv) || misaligned(v) || misaligned(dout)) return NA1D_ERR_ALIGN;
    if (workspace && misaligned(workspace)) return NA1D_ERR_ALIGN;
    if (!(p_drop >= 0.f && p_drop < 1.f)) return NA1D_ERR_SHAPE;
    if (row_stride < 1 || row_offset < 0 || row_offset >= row_stride || seq_rows < row_offset + row_stride * (T - 1) + 1 ||
        seq_rows > 0x7fffffffLL)
        return NA1D_ERR_SHAPE;
    g.drop = na1d::make_dropout(p_drop, seed, (uint32_t)row_stride, (uint32_t)row_offset, (uint32_t)seq_rows);
    na1d::Layout in, outl;
    const int ls = check_layout(qkv_strides, g, in), lo = check_layout(out_strides, g, outl);
    if (ls != NA1D_OK || lo != NA1D_OK) return ls != NA1D_OK ? ls : lo;
    if (!mfma_allowed()) return NA1D_ERR_UNSUPPORTED;
    return mfma_fused_bwd(dq, dk, dv, drpb, q, k, v, nullptr, dout, lse, rpb, t_valid, g, in, outl, scale, dtype,
                          (float *)workspace, workspace ? workspace_bytes : 0, (hipStream_t)stream);
}

int na1d_global_forward(void *out, float *lse, const void *q, const void *k, const void *v, const int32_t *t_valid,
                        int64_t B, int64_t H, int64_t T, int64_t C, float scale, int dtype, float p_drop, uint64_t seed,
                        void *stream) {
    NA1D_CHECK(out, q, k, B, T, C, 1, 0, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!v) return NA1D_ERR_NULL;
    if (misaligned(v)) return NA1D_ERR_ALIGN;
    if (!(p_drop >= 0.f && p_drop < 1.f)) return NA1D_ERR_SHAPE;
    g.drop = na1d::make_dropout(p_drop, seed);
    return na1d::mfma::global_fwd(out, lse, q, k, v, t_valid, g, scale, dtype, (hipStream_t)stream);
}

int na1d_global_backward(void *dq, void *dk, void *dv, const void *q, const void *k, const void *v, const void *out,
                         const void *dout, const float *lse, const int32_t *t_valid, int64_t B, int64_t H, int64_t T,
                         int64_t C, float scale, int dtype, float p_drop, uint64_t seed, void *workspace,
                         int64_t workspace_bytes, void *stream) {
    NA1D_CHECK(dq, q, k, B, T, C, 1, 0, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!dk || !dv || !v || !out || !dout || !lse || !workspace) return NA1D_ERR_NULL;
    if (misaligned(dk) || misaligned(dv) || misaligned(v) || misaligned(out) || misaligned(dout) || misaligned(workspace))
        return NA1D_ERR_ALIGN;
    if (workspace_bytes < g.B * g.T * (int64_t)sizeof(float)) return NA1D_ERR_SHAPE;
    if (!(p_drop >= 0.f && p_drop < 1.f)) return NA1D_ERR_SHAPE;
    g.drop = na1d::make_dropout(p_drop, seed);
    return na1d::mfma::global_bwd(dq, dk, dv, (float *)workspace, q, k, v, out, dout, lse, t_valid, g, scale, dtype,
                                  (hipStream_t)stream);
}

int na1d_fused_backward_noalloc(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
                                const void *out, const void *dout, const float *lse, const float *rpb,
                                const int32_t *t_valid, int64_t B, int64_t H, int64_t T, int64_t C, int64_t W,
                                int64_t left, float scale, int dtype, void *stream) {
    NA1D_CHECK(dq, q, k, B, T, C, W, left, H, dtype, g);
    if (bad_scale(scale)) return NA1D_ERR_SCALE;
    if (!dk || !dv || !v || !out || !dout || !lse) return NA1D_ERR_NULL;
    if (misaligned(dk) || misaligned(dv) || misaligned(v) || misaligned(out) || misaligned(dout))
        return NA1D_ERR_ALIGN;
    if (!mfma_allowed()) return NA1D_ERR_UNSUPPORTED;      // the generic kernels have no fixed-order reduction
    const int64_t need = na1d::mfma::fused_bwd_workspace_bytes(g, dtype);
    if (need <= 0) return NA1D_ERR_UNSUPPORTED;
    if (need > na1d::mfma::kStaticScratchBytes) return NA1D_ERR_TOO_LARGE;
    float *scratch = nullptr;
    const int ss = na1d::mfma::static_scratch(&scratch);
    if (ss != NA1D_OK) return ss;
    const na1d::Layout packed = na1d::packed_layout(g);
    return mfma_fused_bwd(dq, dk, dv, drpb, q, k, v, out, dout, lse, rpb, t_valid, g, packed, packed, scale, dtype, scratch,
                          need, (hipStream_t)stream);
}

int64_t na1d_global_backward_workspace_bytes(int64_t B, int64_t H, int64_t T, int64_t C, int dtype) {
    Geom g;
    const int st = check_shape(B, T, C, 1, 0, H, dtype, g);
    if (st < 0) return st;
    return st > 0 ? 0 : g.B * g.T * (int64_t)sizeof(float);
}

int na1d_force_generic(int on) { return generic_forced().exchange(on ? 1 : 0); }

int na1d_profile_events(void *start, void *stop) {
    na1d::LaunchEvents &ev = na1d::launch_events();
    ev.start = (hipEvent_t)start;
    ev.stop = (hipEvent_t)stop;
    return NA1D_OK;
}

const char *na1d_profile_last_kernel(void) { return na1d::launch_events().kernel; }

int64_t na1d_fused_backward_workspace_bytes(int64_t B, int64_t H, int64_t T, int64_t C, int64_t W, int64_t left,
                                            int dtype) {
    Geom g;
    const int st = check_shape(B, T, C, W, left, H, dtype, g);
    if (st < 0) return st;
    if (st > 0 || !mfma_allowed()) return 0;
    return na1d::mfma::fused_bwd_workspace_bytes(g, dtype);
}

}  // extern "C"
