// Fused NA1D forward and backward on the matrix cores for windows that the two- and
// three-block kernels of na1d_mfma.hip do not cover: W up to 80, or more than 16 keys
// on one side.  Same tiling, LDS layout and operand conventions (na1d_mfma_core.h),
// with NBV = ceil((15 + W) / 16) <= 6 virtual key blocks per query tile and no merging
// of blocks: lane (n, g) carries 4*NBV score slots, slot j = 16*vb + 4g + r - shift - n + L.
#include "na1d_mfma_core.h"

namespace na1d {
namespace mfma {

constexpr int kMaxWideBlocks = 6;
constexpr int kBiasSlots = 96;   // W <= 80, padded

// Blocks and shift of a wide window; 0 blocks if the shape is not covered.
struct WideCover {
    int nbv, shift;
};
inline WideCover wide_cover(const Geom &g) {
    WideCover c{0, 0};
    if (g.C != 16 && g.C != 32 && g.C != 64 && g.C != 128) return c;
    if (g.T > (1 << 29) / g.C || g.W > NA1D_MAX_WINDOW) return c;
    c.nbv = (15 + g.W + 15) / 16;
    if (c.nbv < 3) c.nbv = 3;
    // any shift in [L, 16*NBV - 16 - R] covers the window; prefer one that puts key blocks on 128-byte lines
    const int R = g.W - 1 - g.L, rows = std::max(1, 128 / (2 * g.C));
    const int s = (g.L + rows - 1) / rows * rows;
    c.shift = s <= 16 * c.nbv - 16 - R ? s : g.L;
    return c;
}

// rpb row of this head times log2(e) in LDS slots [0, W); -inf is applied at the read
__device__ inline void stage_bias(LDS_PTR(float) bias_lds, const float *rpb_h, int W, int tid) {
    if (tid < kBiasSlots) bias_lds[tid] = (rpb_h && tid < W) ? rpb_h[tid] * kLog2e : 0.f;
}
__device__ inline float bias_at(LDS_PTR(float) bias_lds, int j, int W) {
    const float val = bias_lds[min(max(j, 0), kBiasSlots - 1)];
    return (j >= 0 && j < W) ? val : kNegInf;
}

// =============================================================================
// Forward
// =============================================================================
template <class DT, int C, int NBV>
__global__ void __launch_bounds__(kThreads)
wide_fwd_kernel(char *__restrict__ out, float *__restrict__ lse, const char *__restrict__ q,
                const char *__restrict__ k, const char *__restrict__ v, const float *__restrict__ rpb,
                const int32_t *__restrict__ t_valid, uint32_t items, int T, int W, int L, int H, int tiles, int nt,
                int strips, float scale, uint32_t strips_magic, uint32_t heads_magic, Strides in, Strides outl,
                int shift) {
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    constexpr int MT = Strip<C>::kMaxTiles;
    fetch_args_now(out, lse, q, k, v, rpb, t_valid, items, T, W, L, H, tiles, nt, strips, scale, strips_magic, heads_magic,
                   in.sample, in.head, in.pitch, outl.sample, outl.head, outl.pitch, shift);
    // dynamic LDS (launch_wide_fwd): K and V regions of kt tiles starting sb tiles before the strip, Q region of nt
    // tiles, kBiasSlots bias floats
    const int sb = (shift + 15) >> 4;                        // whole tiles in front of the strip
    const int kt = nt - 1 + NBV + ((shift & 15) ? 1 : 0);    // tiles a key-side region holds
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int key_region = region_bytes<C>(kt);
    LDS_PTR(char) k_lds = (LDS_PTR(char))smem;
    LDS_PTR(char) v_lds = k_lds + key_region;
    LDS_PTR(char) q_lds = v_lds + key_region;
    LDS_PTR(float) bias_lds = (LDS_PTR(float))(q_lds + region_bytes<C>(nt));

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const WorkItem wi = work_item(blockIdx.x, items, strips, strips_magic, H, heads_magic);
    const uint32_t b = wi.sample * H + wi.head, sample = wi.sample, head = wi.head;
    const int i0 = wi.strip * nt, i1 = min(i0 + nt, tiles);
    const int g = lane >> 4, n = lane & 15;

    const int64_t in_off = sample * in.sample + head * in.head, out_off = sample * outl.sample + head * outl.head;
    const int key_rows = max(0, min(T, 16 * (i0 - sb + kt)));
    const Rsrc qs = make_rsrc(q + in_off, min(T, 16 * i1) * in.pitch), ks = make_rsrc(k + in_off, key_rows * in.pitch);
    const Rsrc vs = make_rsrc(v + in_off, key_rows * in.pitch), os = make_rsrc(out + out_off, T * outl.pitch);
    const Rsrc ls = make_rsrc(lse ? lse + (int64_t)b * T : nullptr, lse ? T * 4 : 0);
    const bool out_whole_lines = stores_whole_lines(outl.pitch, C, 0);
    {
        const int lane_off = direct_lane_offset<C>(wave, lane, in.pitch);
        stage_direct<C, MT + NBV, kReadShared>(ks, 16 * (i0 - sb), k_lds, kt, wave, lane_off, in.pitch);
        stage_direct<C, MT, kReadShared>(qs, 16 * i0, q_lds, nt, wave, lane_off, in.pitch);
        stage_direct<C, MT + NBV, kReadShared>(vs, 16 * (i0 - sb), v_lds, kt, wave, lane_off, in.pitch);
        stage_bias(bias_lds, rpb ? rpb + head * W : nullptr, W, tid);
    }

    int tv = T;
    if (t_valid) tv = max(0, min(T, t_valid[sample]));
    const float scale2 = scale * kLog2e;

    RowLane<C> k_lane, q_lane;
    TrLane<C> v_lane;
    k_lane.init(16 * sb - shift, lane);
    q_lane.init(0, lane);
    v_lane.init(16 * sb - shift, lane);

    wait_direct();
    __syncthreads();
    float bias[NBV][4];
#pragma unroll
    for (int vb = 0; vb < NBV; ++vb)
#pragma unroll
        for (int r = 0; r < 4; ++r) bias[vb][r] = bias_at(bias_lds, 16 * vb + 4 * g + r - shift - n + L, W);

    for (int i = i0 + wave; i < i1; i += kWaves) {
        const int tile_bytes = (i - i0) * LL::kTileBytes;
        RowOperand<C> qt;
        read_rows<C>(qt, q_lds + tile_bytes, q_lane);
        float z[NBV][4];
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            RowOperand<C> kop;
            read_rows<C>(kop, k_lds + tile_bytes + vb * LL::kTileBytes, k_lane);
            const f32x4 s = dot_rows_mma<DT, C>(kop, qt);
#pragma unroll
            for (int r = 0; r < 4; ++r) z[vb][r] = __builtin_fmaf(s[r], scale2, bias[vb][r]);
        }
        const int s0 = 16 * i - shift;           // first row of the window
        const int qrow = 16 * i + n;
        if (s0 < 0 || s0 + 16 * NBV > tv) {      // the model's additive -100, only on tiles that touch an edge
            const bool row_masked = qrow >= tv;
#pragma unroll
            for (int vb = 0; vb < NBV; ++vb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t key = (uint32_t)(s0 + 16 * vb + 4 * g + r);   // unsigned: also key < 0
                    z[vb][r] += (key >= (uint32_t)tv || row_masked) ? kMaskValue * kLog2e : 0.f;
                }
        }
        float m = kNegInf;
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) m = max3(m, max2(z[vb][0], z[vb][1]), max2(z[vb][2], z[vb][3]));
        m = xor_max(m);
        float sum = 0.f;
        u32x2 pb[NBV];
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                p[r] = __builtin_amdgcn_exp2f(z[vb][r] - m);
                sum += p[r];
            }
            pb[vb] = u32x2{Mma<DT>::pack(p[0], p[1]), Mma<DT>::pack(p[2], p[3])};
        }
        sum = xor_sum(sum);
        const float inv = __builtin_amdgcn_rcpf(sum);

        f32x4 o[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            LDS_PTR(char) blk = v_lds + tile_bytes + vb * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) o[ct] = Mma<DT>::k16(read_tr(blk + v_lane.off[ct]), pb[vb], o[ct]);
        }
        u32x2 ow[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) ow[ct] = pack_acc<DT>(o[ct], inv);
        store_tile<C>(os, qrow * outl.pitch, ow, g, out_whole_lines);   // rows past T are dropped by the store
        if (g == 0)
            __builtin_amdgcn_raw_buffer_store_b32(
                __float_as_uint((m + __builtin_amdgcn_logf(sum)) * kLn2), ls, qrow * 4, 0, 0);
    }
}

template <class DT, int C, int NBV>
int launch_wide_fwd_n(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
                      const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &outl, float scale,
                      int shift, hipStream_t s) {
    const Split sp = make_split(g.B, g.T, Strip<C>::kMaxTiles);
    if (!items_ok(sp, g) || !strides_ok(in, g) || !strides_ok(outl, g)) return NA1D_ERR_UNSUPPORTED;
    auto kern = wide_fwd_kernel<DT, C, NBV>;
    const int kt = sp.nt - 1 + NBV + ((shift & 15) ? 1 : 0);
    const size_t lds = (size_t)2 * region_bytes<C>(kt) + region_bytes<C>(sp.nt) + kBiasSlots * sizeof(float);
    if (!allow_lds(kern, lds)) return NA1D_ERR_LAUNCH;
    launch_kernel(kern, (unsigned)sp.items, lds, s, (char *)out, lse, (const char *)q, (const char *)k, (const char *)v,
                  rpb, t_valid, (uint32_t)sp.items, (int)g.T, g.W, g.L, g.H, sp.tiles, sp.nt, sp.strips, scale,
                  div_magic(sp.strips), div_magic(g.H), byte_strides(in), byte_strides(outl), shift);
    return launch_status();
}

template <class DT, int C>
int launch_wide_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
                    const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &outl, float scale,
                    hipStream_t s) {
    const WideCover c = wide_cover(g);
    switch (c.nbv) {
        case 3: return launch_wide_fwd_n<DT, C, 3>(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, c.shift, s);
        case 4: return launch_wide_fwd_n<DT, C, 4>(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, c.shift, s);
        case 5: return launch_wide_fwd_n<DT, C, 5>(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, c.shift, s);
        case 6: return launch_wide_fwd_n<DT, C, 6>(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, c.shift, s);
    }
    return NA1D_ERR_UNSUPPORTED;
}

int wide_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
             const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &outl, float scale, int dtype,
             hipStream_t s) {
    if (!wide_cover(g).nbv) return NA1D_ERR_UNSUPPORTED;
    NA1D_MFMA_DISPATCH(launch_wide_fwd, out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, s);
}

}  // namespace mfma
}  // namespace na1d
