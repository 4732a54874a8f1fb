// Fused NA1D forward and backward on the matrix cores for windows that the two- and
// three-block kernels of na1d_mfma.hip do not cover: W up to 80, or more than 16 keys
// on one side.  Same tiling, LDS layout and operand conventions (na1d_mfma_core.h),
// with NBV = ceil((15 + W) / 16) <= 6 virtual key blocks per query tile and no merging
// of blocks: lane (n, g) carries 4*NBV score slots, slot j = 16*vb + 4g + r - shift - n + L.
#include "na1d_mfma_core.h"

namespace na1d {
namespace mfma {

constexpr int kBiasSlots = 96;   // W <= 80, padded

// Blocks and shift of a wide window; 0 blocks if the shape is not covered.
struct WideCover {
    int nbv, shift;
};
inline WideCover wide_cover(const Geom &g) {
    WideCover c{0, 0};
    if (g.C > 128) return c;             // head_dim is run at the next of 16, 32, 64, 128, zero-padded
    if (g.T > (1 << 29) / g.C || g.W > NA1D_MAX_WINDOW) return c;
    c.nbv = (15 + g.W + 15) / 16;
    if (c.nbv < 3) c.nbv = 3;
    // any shift in [L, 16*NBV - 16 - R] covers the window; prefer one that puts key blocks on 128-byte lines
    const int R = g.W - 1 - g.L, rows = std::max(1, 128 / (2 * g.C));
    const int hi = 16 * c.nbv - 16 - R, s16 = (g.L + 15) / 16 * 16, s = (g.L + rows - 1) / rows * rows;
    c.shift = s16 <= hi ? s16 : s <= hi ? s : g.L;      // whole tiles, else whole lines, else the first key
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
template <class DT, int C, int NBV, bool DROP>
__global__ void __launch_bounds__(kThreads)
wide_fwd_kernel(char *__restrict__ out, float *__restrict__ lse, const char *__restrict__ q,
                const char *__restrict__ k, const char *__restrict__ v, const float *__restrict__ rpb,
                const int32_t *__restrict__ t_valid, uint32_t items, int T, int W, int L, int H, int tiles, int nt,
                int strips, float scale, uint32_t strips_magic, uint32_t heads_magic, Strides in, Strides outl,
                int shift, Dropout drop) {
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    constexpr int MT = Strip<C>::kMaxTiles;
    fetch_args_now(out, lse, q, k, v, rpb, t_valid, items, T, W, L, H, tiles, nt, strips, scale, strips_magic, heads_magic,
                   in.sample, in.head, in.pitch, in.width, outl.sample, outl.head, outl.pitch, outl.width, shift);
    if constexpr (DROP) fetch_args_now(drop.threshold, drop.seed_lo, drop.seed_hi, drop.inv_keep, drop.row_stride, drop.row_offset, drop.seq_rows);
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
        const int lane_off = direct_lane_offset<C>(wave, lane, in.pitch, in.width);
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
    barrier_lds();
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
        const uint32_t drop_key = DROP ? dropout_row_key(dropout_row(drop, b, T, qrow), drop) : 0u;
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                p[r] = __builtin_amdgcn_exp2f(z[vb][r] - m);
                sum += p[r];
                // a dropped probability stays in the sum and leaves O
                if (DROP && !dropout_keeps(drop_key, 16 * vb + 4 * g + r - shift - n + L, drop)) p[r] = 0.f;
            }
            pb[vb] = u32x2{Mma<DT>::pack(p[0], p[1]), Mma<DT>::pack(p[2], p[3])};
        }
        sum = xor_sum(sum);
        const float inv = __builtin_amdgcn_rcpf(sum) * (DROP ? drop.inv_keep : 1.f);

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
        store_tile<C>(os, qrow * outl.pitch, ow, g, out_whole_lines, outl.width);   // rows past T are dropped by the store
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
    auto kern = g.drop.threshold ? wide_fwd_kernel<DT, C, NBV, true> : wide_fwd_kernel<DT, C, NBV, false>;
    const int kt = sp.nt - 1 + NBV + ((shift & 15) ? 1 : 0);
    const size_t lds = (size_t)2 * region_bytes<C>(kt) + region_bytes<C>(sp.nt) + kBiasSlots * sizeof(float);
    if (!allow_lds(kern, lds)) return NA1D_ERR_LAUNCH;
    note_kernel("wide_fwd_kernel", DT::tag, C, NBV, g.drop.threshold != 0);
    launch_kernel(kern, (unsigned)sp.items, lds, s, (char *)out, lse, (const char *)q, (const char *)k, (const char *)v,
                  rpb, t_valid, (uint32_t)sp.items, (int)g.T, g.W, g.L, g.H, sp.tiles, sp.nt, sp.strips, scale,
                  div_magic(sp.strips), div_magic(g.H), byte_strides(in, g), byte_strides(outl, g), shift, g.drop);
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

// =============================================================================
// Backward
// =============================================================================
// Same two passes as the two/three-block backward (na1d_mfma.hip), with the halo sized by the window: key block
// kp (rows 16*kp - shift ...) is virtual block vb of query tile kp - vb, so the key blocks that touch the strip's
// rows need the query tiles i0 - HB .. i1 - 1 + HA with HB = NBV - 1 - floor(shift / 16) and HA = ceil(shift / 16).
// A strip is at most kWideQueryTiles - HB - HA tiles long so that a wave keeps the rounded P and dS of its two query
// tiles in registers until the K/V regions can be reused for them.
constexpr int kWideQueryTiles = 8;
constexpr int kWideTPW = kWideQueryTiles / kWaves;
constexpr int kWideSlots = 128;          // d rpb slot sums per wave: slot + 32 indexes them
static_assert(kWideQueryTiles * 16 <= kThreads, "one lane per staged lse row");

struct WideBwdShape {
    int hb, ha, mt;                      // halo query tiles before / after, strip length
    int kx;                              // key blocks that touch a strip's rows beyond one per tile: 1 unless shift % 16 == 0
};
inline WideBwdShape wide_bwd_shape(const WideCover &c) {
    WideBwdShape w;
    w.hb = c.nbv - 1 - (c.shift >> 4);
    w.ha = (c.shift + 15) >> 4;
    w.mt = kWideQueryTiles - w.hb - w.ha;
    w.kx = w.ha - (c.shift >> 4);
    return w;
}

template <class DT, int C, int NBV, bool DROP>
__global__ void __launch_bounds__(kThreads)
wide_bwd_kernel(char *__restrict__ dq, char *__restrict__ dk, char *__restrict__ dv, float *__restrict__ drpb,
                const char *__restrict__ q, const char *__restrict__ k, const char *__restrict__ v,
                const char *__restrict__ dout, const float *__restrict__ lse, const float *__restrict__ rpb,
                const int32_t *__restrict__ t_valid, uint32_t items, int T, int W, int L, int H, int tiles, int nt,
                int strips, float scale, float *__restrict__ drpb_partial, int kv_bytes, uint32_t strips_magic,
                uint32_t heads_magic, Strides in, Strides outl, int shift, Dropout drop) {
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    constexpr int kScoreTile = 16 * 16 * 2;                // one 16x16 tile of 16-bit scores
    fetch_args_now(dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, items, T, W, L, H, tiles, nt, strips, scale,
                   drpb_partial, kv_bytes, strips_magic, heads_magic, in.sample, in.head, in.pitch, in.width, outl.sample,
                   outl.head, outl.pitch, outl.width, shift);
    if constexpr (DROP) fetch_args_now(drop.threshold, drop.seed_lo, drop.seed_hi, drop.inv_keep, drop.row_stride, drop.row_offset, drop.seq_rows);
    const int hb = NBV - 1 - (shift >> 4), ha = (shift + 15) >> 4;
    const int qtiles = nt + hb + ha;                        // query-side tiles, <= kWideQueryTiles
    const int ktiles = qtiles + NBV - 1;                    // key-side tiles: whole virtual blocks
    // dynamic LDS (launch_wide_bwd): [K region | V region] starting at the first key of query tile i0 - hb, reused
    // after pass 1 for the score tiles of the strip's key blocks [((kp - kp_lo) * NBV + vb) * 2 + P/dS] and padded to kv_bytes; Q, dO regions of qtiles
    // tiles; lse of the query-side rows; bias; d rpb slot sums per wave
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int key_region = region_bytes<C>(ktiles), qry_region = region_bytes<C>(qtiles);
    LDS_PTR(char) k_lds = (LDS_PTR(char))smem;
    LDS_PTR(char) v_lds = k_lds + key_region;
    LDS_PTR(char) sc_lds = k_lds;
    LDS_PTR(char) q_lds = k_lds + kv_bytes;
    LDS_PTR(char) g_lds = q_lds + qry_region;               // dO
    LDS_PTR(float) lse_lds = (LDS_PTR(float))(g_lds + qry_region);
    LDS_PTR(float) bias_lds = lse_lds + kThreads;
    LDS_PTR(float) rsum = bias_lds + kBiasSlots;            // [kWaves][kWideSlots]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const WorkItem wi = work_item(blockIdx.x, items, strips, strips_magic, H, heads_magic);
    const uint32_t item = wi.item, b = wi.sample * H + wi.head, sample = wi.sample, head = wi.head;
    const int i0 = wi.strip * nt, i1 = min(i0 + nt, tiles);
    const int g = lane >> 4, n = lane & 15;
    const int q0 = i0 - hb;                                 // first query-side tile

    const int64_t in_off = sample * in.sample + head * in.head, out_off = sample * outl.sample + head * outl.head;
    {
        const int key_rows = max(0, min(T, 16 * (q0 + ktiles) - shift));
        const int qry_rows = max(0, min(T, 16 * (q0 + qtiles)));
        const Rsrc ks = make_rsrc(k + in_off, key_rows * in.pitch), vs = make_rsrc(v + in_off, key_rows * in.pitch);
        const Rsrc qs = make_rsrc(q + in_off, qry_rows * in.pitch), gs = make_rsrc(dout + out_off, qry_rows * outl.pitch);
        const Rsrc ls = make_rsrc(lse + (int64_t)b * T, T * 4);
        const int lane_off = direct_lane_offset<C>(wave, lane, in.pitch, in.width);
        const int lane_off_g = direct_lane_offset<C>(wave, lane, outl.pitch, outl.width);
        load_to_lds<4, 0>(ls, (LDS_PTR(char))(lse_lds + 64 * wave), (16 * q0 + tid) * 4);
        constexpr int KT = kWideQueryTiles + NBV - 1;
        stage_direct<C, KT, kReadShared>(ks, 16 * q0 - shift, k_lds, ktiles, wave, lane_off, in.pitch);
        stage_direct<C, kWideQueryTiles, kReadShared>(qs, 16 * q0, q_lds, qtiles, wave, lane_off, in.pitch);
        stage_direct<C, KT, kReadShared>(vs, 16 * q0 - shift, v_lds, ktiles, wave, lane_off, in.pitch);
        stage_direct<C, kWideQueryTiles, kReadShared>(gs, 16 * q0, g_lds, qtiles, wave, lane_off_g, outl.pitch);
        stage_bias(bias_lds, rpb ? rpb + head * W : nullptr, W, tid);
    }

    int tv = T;
    if (t_valid) tv = max(0, min(T, t_valid[sample]));
    const float scale2 = scale * kLog2e;
    const float mask2 = kMaskValue * kLog2e;

    RowLane<C> row_lane;                // row operands (virtual key blocks and query tiles are whole tiles)
    TrLane<C> tr_lane;                  // transposed operands of the same
    row_lane.init(0, lane);
    tr_lane.init(0, lane);

    wait_direct();
    barrier_lds();
    float bias[NBV][4];
#pragma unroll
    for (int vb = 0; vb < NBV; ++vb)
#pragma unroll
        for (int r = 0; r < 4; ++r) bias[vb][r] = bias_at(bias_lds, 16 * vb + 4 * g + r - shift - n + L, W);

    // ---------------- pass 1: query tiles q0 .. q0 + qtiles - 1 -> dQ, d rpb, score tiles ----------------
    float racc[NBV][4];
#pragma unroll
    for (int vb = 0; vb < NBV; ++vb)
#pragma unroll
        for (int r = 0; r < 4; ++r) racc[vb][r] = 0.f;
    const Rsrc dqs = make_rsrc(dq + in_off, T * in.pitch);
    const bool dq_whole_lines = stores_whole_lines(in.pitch, C, 0);
    u32x2 sc[kWideTPW][NBV][2];         // [tile of this wave][block][P / dS], rounded to 16 bit
#pragma unroll
    for (int jt = 0; jt < kWideTPW; ++jt) {
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) sc[jt][vb][0] = sc[jt][vb][1] = u32x2{0u, 0u};
        const int tq = wave + jt * kWaves;                  // tile index inside the query-side regions
        const int qt = q0 + tq;
        if (tq >= qtiles || qt < 0 || qt >= tiles) continue;   // nothing there: its scores stay zero
        RowOperand<C> qop, gop;
        read_rows<C>(qop, q_lds + tq * LL::kTileBytes, row_lane);
        read_rows<C>(gop, g_lds + tq * LL::kTileBytes, row_lane);
        const float lse2 = lse_lds[tq * 16 + n] * kLog2e;
        const int s0 = 16 * qt - shift;
        const int qrow = 16 * qt + n;
        const bool edge = s0 < 0 || s0 + 16 * NBV > tv;
        float p[NBV][4], dp[NBV][4], part = 0.f;
        // With dropout mask D (0 or 1/(1-p)): O = (D*P) V, so dV takes D*P and dP = D * (dO . V^T).
        const uint32_t drop_key = DROP ? dropout_row_key(dropout_row(drop, b, T, qrow), drop) : 0u;
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            RowOperand<C> kop, vop;
            const int off = (tq + vb) * LL::kTileBytes;
            read_rows<C>(kop, k_lds + off, row_lane);
            read_rows<C>(vop, v_lds + off, row_lane);
            const f32x4 s = dot_rows_mma<DT, C>(kop, qop);
            const f32x4 d = dot_rows_mma<DT, C>(vop, gop);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float z = __builtin_fmaf(s[r], scale2, bias[vb][r]) - lse2;
                if (edge) {
                    const uint32_t key = (uint32_t)(s0 + 16 * vb + 4 * g + r);   // unsigned: also key < 0
                    z += (key >= (uint32_t)tv || qrow >= tv) ? mask2 : 0.f;
                }
                p[vb][r] = __builtin_amdgcn_exp2f(z);
                dp[vb][r] = d[r];
                if constexpr (DROP)
                    dp[vb][r] *= dropout_keeps(drop_key, 16 * vb + 4 * g + r - shift - n + L, drop) ? drop.inv_keep : 0.f;
                part = __builtin_fmaf(p[vb][r], dp[vb][r], part);
            }
        }
        const float delta = xor_sum(part);
        const bool own = qt >= i0 && qt < i1;               // halo tiles only contribute their scores
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            float ds[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                ds[r] = p[vb][r] * (dp[vb][r] - delta);
                if (own) racc[vb][r] += ds[r];
                if constexpr (DROP)        // the probability as the forward used it
                    p[vb][r] *= dropout_keeps(drop_key, 16 * vb + 4 * g + r - shift - n + L, drop) ? drop.inv_keep : 0.f;
            }
            sc[jt][vb][0] = u32x2{Mma<DT>::pack(p[vb][0], p[vb][1]), Mma<DT>::pack(p[vb][2], p[vb][3])};
            sc[jt][vb][1] = u32x2{Mma<DT>::pack(ds[0], ds[1]), Mma<DT>::pack(ds[2], ds[3])};
        }
        if (!own) continue;
        f32x4 acc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            LDS_PTR(char) blk = k_lds + (tq + vb) * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) acc[ct] = Mma<DT>::k16(read_tr(blk + tr_lane.off[ct]), sc[jt][vb][1], acc[ct]);
        }
        u32x2 qw[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) qw[ct] = pack_acc<DT>(acc[ct], scale);
        store_tile<C>(dqs, qrow * in.pitch, qw, g, dq_whole_lines, in.width);
    }

    // d rpb.  Register (vb, r) of lane (n, g) holds key a = 4g + r of block vb against query n: slot
    // 16*vb + a - n + L - shift.  A lane permutation lines the diagonals a - n = d (mod 16) up in lane d; members
    // with a >= d have a - n = d, the others d - 16, i.e. the slot of the block before.  Lane d thus owns the
    // slots d + L - shift + 16*k, k = -1 .. NBV-1; the four lane groups hold the same sums and share the stores.
    if (drpb) {
        float up[NBV], lo[NBV];
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) up[vb] = lo[vb] = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int a = 4 * g + r;
            const int from = (16 * g + ((a - n) & 15)) * 4;
            const bool upper = a >= n;
#pragma unroll
            for (int vb = 0; vb < NBV; ++vb) {
                const float y = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(racc[vb][r])));
                up[vb] += upper ? y : 0.f;
                lo[vb] += upper ? 0.f : y;
            }
        }
        LDS_PTR(float) mine = rsum + wave * kWideSlots + 32 + (n + L - shift);
#pragma unroll
        for (int kk = -1; kk < NBV; ++kk) {                 // slot n + L - shift + 16*kk
            float t = (kk >= 0 ? up[kk >= 0 ? kk : 0] : 0.f) + (kk + 1 < NBV ? lo[kk + 1 < NBV ? kk + 1 : 0] : 0.f);
            t = xor_sum(t);
            if (g == ((kk + 1) & 3)) mine[16 * kk] = t;
        }
    }

    // Pass 2 reads the score tiles of the key blocks that touch the strip's rows, kp_lo .. kp_hi: block vb of query
    // tile tq is key block q0 + tq + vb, and only those in the range are kept (about half of what pass 1 computed).
    const int kp_lo = i0 + (shift >> 4), kp_hi = i1 - 1 + ha;
    barrier_lds();                      // every wave is done with K and V: their regions become the score tiles
#pragma unroll
    for (int jt = 0; jt < kWideTPW; ++jt) {
        const int tq = wave + jt * kWaves;
        if (tq >= qtiles) continue;
        LDS_PTR(char) t = sc_lds + n * 32 + g * 8;          // tile[query n][key slots 4g..4g+3]
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            const int kp = q0 + tq + vb;
            if (kp < kp_lo || kp > kp_hi) continue;
#pragma unroll
            for (int pd = 0; pd < 2; ++pd)
                *reinterpret_cast<LDS_PTR(u32x2)>(t + (((kp - kp_lo) * NBV + vb) * 2 + pd) * kScoreTile) = sc[jt][vb][pd];
        }
    }
    barrier_lds();

    // ---------------- pass 2: key blocks of the strip -> dK, dV ----------------
    const int sc_lane = (4 * g + (n >> 2)) * 32 + (n & 3) * 8;       // transposed read of a score tile
    const int row_lo = 16 * i0, row_hi = min(T, 16 * i1);            // rows this strip owns
    const Rsrc dks = make_rsrc(dk + in_off + (int64_t)row_lo * in.pitch, (row_hi - row_lo) * in.pitch);
    const Rsrc dvs = make_rsrc(dv + in_off + (int64_t)row_lo * in.pitch, (row_hi - row_lo) * in.pitch);
    const bool whole_lines = stores_whole_lines(in.pitch, C, shift);
    for (int kp = kp_lo + wave; kp <= kp_hi; kp += kWaves) {
        f32x4 acck[CT], accv[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acck[ct] = accv[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            const int tq = kp - vb - q0;                    // in [0, qtiles) by the choice of hb and ha
            LDS_PTR(char) qtile = q_lds + tq * LL::kTileBytes;
            LDS_PTR(char) gtile = g_lds + tq * LL::kTileBytes;
            LDS_PTR(char) stile = sc_lds + ((kp - kp_lo) * NBV + vb) * 2 * kScoreTile + sc_lane;
            const u32x2 pb = read_tr(stile), db = read_tr(stile + kScoreTile);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                accv[ct] = Mma<DT>::k16(read_tr(gtile + tr_lane.off[ct]), pb, accv[ct]);
                acck[ct] = Mma<DT>::k16(read_tr(qtile + tr_lane.off[ct]), db, acck[ct]);
            }
        }
        const int row_off = (16 * (kp - i0) - shift + n) * in.pitch;    // outside the strip -> dropped
        u32x2 kw[CT], vw[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            kw[ct] = pack_acc<DT>(acck[ct], scale);
            vw[ct] = pack_acc<DT>(accv[ct], 1.f);
        }
        store_tile<C>(dks, row_off, kw, g, whole_lines, in.width);
        store_tile<C>(dvs, row_off, vw, g, whole_lines, in.width);
    }

    if (drpb && tid < W) {              // rsum was complete at the barriers before pass 2
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) t += rsum[w * kWideSlots + 32 + tid];
        if (drpb_partial)
            drpb_partial[(size_t)item * kWidePartialStride + tid] = t;   // folded by drpb_reduce_kernel
        else
            atomicAdd(drpb + head * W + tid, t);
    }
}

// LDS of a workgroup whose strip is nt tiles long, and the K/V part of it
template <int C>
inline size_t wide_bwd_lds(int nt, int nbv, const WideBwdShape &w, int &kv_bytes) {
    const int qtiles = nt + w.hb + w.ha, ktiles = qtiles + nbv - 1;
    kv_bytes = std::max(2 * region_bytes<C>(ktiles), (nt + w.kx) * nbv * 2 * 512);    // K and V, later the score tiles pass 2 reads
    return (size_t)kv_bytes + (size_t)2 * region_bytes<C>(qtiles) +
           (kThreads + kBiasSlots + kWaves * kWideSlots) * sizeof(float);
}

// The split of a wide backward into workgroups: strips as long as a CU's LDS allows.
template <int C>
inline bool wide_bwd_split(const Geom &g, const WideCover &c, Split &sp, int &kv_bytes, size_t &lds) {
    const WideBwdShape w = wide_bwd_shape(c);
    int mt = w.mt;
    while (mt >= 1 && wide_bwd_lds<C>(mt, c.nbv, w, kv_bytes) > 160 * 1024) --mt;   // LDS of one CU
    if (mt < 1) return false;
    sp = make_split(g.B, g.T, mt);
    lds = wide_bwd_lds<C>(sp.nt, c.nbv, w, kv_bytes);
    return true;
}

template <class DT, int C, int NBV>
int launch_wide_bwd_n(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
                      const void *dout, const float *lse, const float *rpb, const int32_t *t_valid, const Geom &g,
                      const Layout &in, const Layout &outl, float scale, const WideCover &c, float *workspace,
                      int64_t workspace_bytes, hipStream_t s) {
    Split sp;
    int kv_bytes = 0;
    size_t lds = 0;
    if (!wide_bwd_split<C>(g, c, sp, kv_bytes, lds)) return NA1D_ERR_UNSUPPORTED;
    if (!items_ok(sp, g) || !strides_ok(in, g) || !strides_ok(outl, g)) return NA1D_ERR_UNSUPPORTED;
    float *partial = nullptr;          // as in the two/three-block backward: a workspace is used or refused
    if (drpb && workspace) {
        if (workspace_bytes < sp.items * kWidePartialStride * (int64_t)sizeof(float)) return NA1D_ERR_WORKSPACE;
        partial = workspace;
    }
    auto kern = g.drop.threshold ? wide_bwd_kernel<DT, C, NBV, true> : wide_bwd_kernel<DT, C, NBV, false>;
    if (!allow_lds(kern, lds)) return NA1D_ERR_LAUNCH;
    note_kernel("wide_bwd_kernel", DT::tag, C, NBV, g.drop.threshold != 0);
    launch_kernel(kern, (unsigned)sp.items, lds, s, (char *)dq, (char *)dk, (char *)dv, drpb, (const char *)q,
                  (const char *)k, (const char *)v, (const char *)dout, lse, rpb, t_valid, (uint32_t)sp.items, (int)g.T,
                  g.W, g.L, g.H, sp.tiles, sp.nt, sp.strips, scale, partial, kv_bytes, div_magic(sp.strips), div_magic(g.H),
                  byte_strides(in, g), byte_strides(outl, g), c.shift, g.drop);
    if (partial && drpb && !launch_events().refused)
        drpb_reduce_kernel<kWidePartialStride><<<(unsigned)(g.H * g.W), 128, 0, s>>>(drpb, partial, (int)(g.B / g.H), g.H,
                                                                                     sp.strips, g.W);
    return launch_status();
}

template <class DT, int C>
int launch_wide_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
                    const void *dout, const float *lse, const float *rpb, const int32_t *t_valid, const Geom &g,
                    const Layout &in, const Layout &outl, float scale, float *workspace, int64_t workspace_bytes,
                    hipStream_t s) {
    const WideCover c = wide_cover(g);
    switch (c.nbv) {
        case 3: return launch_wide_bwd_n<DT, C, 3>(dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, g, in, outl, scale, c, workspace, workspace_bytes, s);
        case 4: return launch_wide_bwd_n<DT, C, 4>(dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, g, in, outl, scale, c, workspace, workspace_bytes, s);
        case 5: return launch_wide_bwd_n<DT, C, 5>(dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, g, in, outl, scale, c, workspace, workspace_bytes, s);
        case 6: return launch_wide_bwd_n<DT, C, 6>(dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, g, in, outl, scale, c, workspace, workspace_bytes, s);
    }
    return NA1D_ERR_UNSUPPORTED;
}

// d rpb: float atomics, or - given a workspace of wide_bwd_workspace_bytes() - per-workgroup partial rows that a second
// kernel folds in a fixed order.
int wide_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v, const void *dout,
             const float *lse, const float *rpb, const int32_t *t_valid, const Geom &g, const Layout &in,
             const Layout &outl, float scale, int dtype, float *workspace, int64_t workspace_bytes, hipStream_t s) {
    if (!wide_cover(g).nbv) return NA1D_ERR_UNSUPPORTED;
    NA1D_MFMA_DISPATCH(launch_wide_bwd, dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, g, in, outl, scale, workspace,
                       workspace_bytes, s);
}

template <int C> int64_t wide_workspace(const Geom &g, const WideCover &c) {
    Split sp;
    int kv_bytes = 0;
    size_t lds = 0;
    if (!wide_bwd_split<C>(g, c, sp, kv_bytes, lds)) return 0;
    return sp.items * kWidePartialStride * (int64_t)sizeof(float);
}
int64_t wide_bwd_workspace_bytes(const Geom &g) {
    const WideCover c = wide_cover(g);
    if (!c.nbv) return 0;
    switch (padded_width(g.C)) {
        case 16: return wide_workspace<16>(g, c);
        case 32: return wide_workspace<32>(g, c);
        case 64: return wide_workspace<64>(g, c);
        case 128: return wide_workspace<128>(g, c);
    }
    return 0;
}

}  // namespace mfma
}  // namespace na1d
