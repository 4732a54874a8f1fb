// Fused NA1D forward and backward on the matrix cores (gfx950).  Tiling, LDS layout and
// operand conventions are described at the top of na1d_mfma_core.h.
#include <mutex>

#include "na1d_mfma_core.h"

namespace na1d {
namespace mfma {

// =============================================================================
// Fused forward
// =============================================================================
constexpr int kGroupTiles = 4;               // tiles per strip when heads are staged in groups
constexpr int kGroupWaves = 8;               // waves per workgroup when heads are staged in groups: a group's regions are
                                             // 2-4 times a head's, and twice the waves keep as many tiles in flight per CU

// HG heads whose rows lie side by side in memory (a projection's output, head h of a token right behind head h-1)
// can be staged together: the strip copies then move HG * C channels of a row in one piece - whole 128-byte lines
// for four heads of 16 channels, where a head alone would ask for quarter lines - into regions laid out as rows of
// C * HG channels, and every wave computes the tiles of one head (kGroupWaves / HG waves share a head's tiles).
// ONE: one head per workgroup (HG == 1) and the strip is the whole sequence.  Nothing is shared with another workgroup
// then, and what a workgroup works out before its first copy can go - strip arithmetic, the XCD-aware order - is cut to
// the sample / head split and three buffer resources: at T around 100 a launch is one round of workgroups, and every
// instruction in front of the first copy is in the launch's duration (6 ns apiece, measured by adding some).
// ONE == 2: such strips of packed rows as wide as the kernel's C (pitch = width = 2*C bytes, in and out): pitch, LDS
// layout (regions for the most tiles a strip can have) and the copies' chunk counts become constants as well.
template <class DT, int C, int NBV, bool DROP, int HG, int ONE>
__global__ void __launch_bounds__(64 * (HG > 1 ? kGroupWaves : kWaves))
fused_fwd_kernel(char *__restrict__ out, float *__restrict__ lse, const char *__restrict__ q,
                 const char *__restrict__ k, const char *__restrict__ v, const float *__restrict__ rpb,
                 const int32_t *__restrict__ t_valid, uint32_t items, int T, int W, int L, int H, int tiles, int nt,
                 int strips, float scale, uint32_t strips_magic, uint32_t heads_magic, Strides in, Strides outl,
                 int shift_arg, Dropout drop) {
    const int shift = NBV == 3 ? 16 : shift_arg;     // three key blocks always start one tile before the query tile
    constexpr int CS = C * HG;                       // channels of a staged row
    constexpr int NW = HG > 1 ? kGroupWaves : kWaves; // waves of the workgroup
    using LL = Lds<CS>;
    constexpr int CT = C / 16;                       // channel tiles of the output
    constexpr int MT = HG > 1 ? kGroupTiles : Strip<CS>::kMaxTiles;
    static_assert(NW % HG == 0, "whole waves per head");
    static_assert(!ONE || HG == 1, "the whole-sequence form is for single heads");
    constexpr bool PK = ONE == 2;
    fetch_args_now(out, lse, q, k, v, rpb, t_valid, items, T, W, L, H, tiles, nt, strips, scale, strips_magic, heads_magic,
                   in.sample, in.head, in.pitch, in.width, outl.sample, outl.head, outl.pitch, outl.width, shift_arg);
    if constexpr (DROP) fetch_args_now(drop.threshold, drop.seed_lo, drop.seed_hi, drop.inv_keep, drop.row_stride, drop.row_offset, drop.seq_rows);
    // dynamic LDS (launch_fwd): K and V regions of nt+2 tiles starting one tile before the strip (row 16*i0 - 16:
    // copies that start on a tile boundary measured faster here than ones that start at the first key, and the
    // forward is not short of LDS), Q region of nt tiles
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int key_region = region_bytes<CS>(PK ? MT + 2 : nt + 2);
    LDS_PTR(char) k_lds = (LDS_PTR(char))smem;
    LDS_PTR(char) v_lds = k_lds + key_region;
    LDS_PTR(char) q_lds = v_lds + key_region;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    LDS_PTR(float) bias_lds = (LDS_PTR(float))(q_lds + region_bytes<CS>(PK ? MT : nt)) + (HG > 1 ? wave % HG : 0) * kBiasEntries;   // the bias table of this wave's head
    const int hw = HG > 1 ? wave % HG : 0;           // this wave's head inside the group
    uint32_t sample, head0, lin_pk = 0;
    int i0, i1;
    if constexpr (PK) {
        lin_pk = blockIdx.x;
        sample = div_by(lin_pk, H, heads_magic);
        head0 = lin_pk - sample * H;
        i0 = 0;
        i1 = tiles;
    } else if constexpr (ONE != 0) {
        // heads that interleave in memory share lines: their workgroups stay on one XCD, behind one L2 (xcd_item);
        // packed rows are nobody else's, and the plain order is 3 % faster
        const uint32_t lin = in.pitch == 2 * C && outl.pitch == 2 * C ? blockIdx.x : xcd_item(blockIdx.x, items);
        sample = div_by(lin, H, heads_magic);
        head0 = lin - sample * H;
        i0 = 0;
        i1 = tiles;
    } else {
        const WorkItem wi = work_item(blockIdx.x, items, strips, strips_magic, H / HG, heads_magic);
        sample = wi.sample;
        head0 = wi.head * HG;
        i0 = wi.strip * nt;
        i1 = min(i0 + nt, tiles);
    }
    const uint32_t head = head0 + hw, b = sample * H + head;
    const int g = lane >> 4, n = lane & 15;

    // resources end with the strip (plus its halo), so the fixed-size copy below
    // fetches nothing beyond what this strip needs
    // first what the strip copies need, and nothing else: a workgroup's life starts with the time to its first copy
    const int in_pitch = PK ? 2 * C : in.pitch;
    const int64_t in_off = PK ? (int64_t)((uint64_t)lin_pk * (uint32_t)(T * 2 * C)) : sample * in.sample + head0 * in.head;
    const int key_bytes = (ONE ? T : min(T, 16 * (i1 + 1))) * in_pitch, qry_bytes = (ONE ? T : min(T, 16 * i1)) * in_pitch;
    const Rsrc qs = make_rsrc(q + in_off, qry_bytes), ks = make_rsrc(k + in_off, key_bytes);
    const Rsrc vs = make_rsrc(v + in_off, key_bytes);

    // stage the strip: K and V rows [16*i0 - 16, 16*i0 + 16*(MT+1)), Q rows [16*i0, 16*i0 + 16*MT)
    constexpr int TW = NW / HG;                      // tiles the workgroup computes side by side
    if constexpr (PK) {
        const int lane_off = direct_lane_offset<CS>(wave, lane);
        stage_packed<CS, MT + 2, kReadOnce, NW>(ks, -16, k_lds, wave, lane_off);
        stage_packed<CS, MT, kReadOnce, NW>(qs, 0, q_lds, wave, lane_off);
        stage_packed<CS, MT + 2, kReadOnce, NW>(vs, -16, v_lds, wave, lane_off);
    } else {
        const int lane_off = direct_lane_offset<CS>(wave, lane, in.pitch, HG * in.width);
        const bool whole_lines = in.pitch == 2 * C || CS % 64 == 0;
        auto stage = [&](auto key_aux, auto qry_aux) {
            constexpr int KA = decltype(key_aux)::value, QA = decltype(qry_aux)::value;
            stage_direct<CS, MT + 2, KA, NW>(ks, 16 * i0 - 16, k_lds, nt + 2, wave, lane_off, in.pitch);
            stage_direct<CS, MT, QA, NW>(qs, 16 * i0, q_lds, nt, wave, lane_off, in.pitch);
            stage_direct<CS, MT + 2, KA, NW>(vs, 16 * i0 - 16, v_lds, nt + 2, wave, lane_off, in.pitch);
        };
        using Once = std::integral_constant<int, kReadOnce>;
        using Shared = std::integral_constant<int, kReadShared>;
        if ((ONE || strips == 1) && whole_lines)         // nobody else reads these rows' lines
            stage(Once{}, Once{});
        else if (!ONE && whole_lines)
            stage(Shared{}, Once{});
        else
            stage(Shared{}, Shared{});
    }
    __builtin_amdgcn_sched_barrier(0);       // the copies are on their way: everything else is worked out behind them
    BiasTable bias_raw;                      // (the wait for the copies covers this load too, wherever it is issued)
    load_bias_table(bias_raw, rpb ? rpb + head * W : nullptr, W, lane);
    const int out_pitch = PK ? 2 * C : outl.pitch, out_width = PK ? 2 * C : outl.width;
    const int64_t out_off = PK ? in_off : sample * outl.sample + head * outl.head;
    const Rsrc os = make_rsrc(out + out_off, T * out_pitch);
    const Rsrc ls = make_rsrc(lse ? lse + (int64_t)b * T : nullptr, lse ? T * 4 : 0);
    const bool out_whole_lines = stores_whole_lines(out_pitch, C, 0);
    const bool out_grouped = HG > 1 && outl.head == 2 * C && outl.width == 2 * C && outl.pitch >= HG * 2 * C;

    int tv = T;
    if (t_valid) tv = max(0, min(T, load_uniform_i32(t_valid, sample)));
    // The matrix core adds the bias for nothing: accumulators start at rpb / scale (-inf outside the window), so
    // x = q.k + rpb / scale comes out of the instruction, z = x * scale * log2(e) is the logit in the log2 domain,
    // and exp2(z - max z) is one multiply-add per slot on the way into the exponential (scale > 0).
    const float scale2 = scale * kLog2e;
    const float inv_scale = __builtin_amdgcn_rcpf(scale);

    // per-lane LDS offsets; key-side regions start 16 rows before the strip
    const int slot = wave / HG;
    RowLane<C, CS> k_lane, q_lane;
    TrLane<C, CS> v_lane;
    k_lane.init(16 - shift, lane, hw * 2 * C);
    q_lane.init(0, lane, hw * 2 * C);
    v_lane.init(16 - shift, lane, hw * 2 * C);
    LDS_PTR(char) k_mine = k_lds + slot * LL::kTileBytes;      // this wave's first tile in each region
    LDS_PTR(char) v_mine = v_lds + slot * LL::kTileBytes;
    LDS_PTR(char) q_mine = q_lds + slot * LL::kTileBytes;

    const uint32_t one2 = DT::tag == NA1D_BF16 ? 0x3f803f80u : 0x3c003c00u;
    const u32x2 ones = {one2, one2};                 // a 16 x 16 block of ones as a matrix operand
    // everything that depends on the lane alone is worked out while the copies are in flight
#pragma unroll
    for (int s_ = 0; s_ < (RowOperand<C>::k32 > 0 ? RowOperand<C>::k32 : 1); ++s_) {
        settle(k_lane.off32[s_]);
        settle(q_lane.off32[s_]);
    }
    settle(k_lane.off16);
    settle(q_lane.off16);
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) settle(v_lane.off[ct]);

    wait_direct();
    wait_bias(bias_raw);
    write_bias_table(bias_lds, bias_raw, W, lane, inv_scale);
    Window<NBV> win;
    read_window<NBV>(win, bias_lds, L, shift, g, n);
    barrier_lds();

    const f32x4 bias_x = {win.bias_x[0], win.bias_x[1], win.bias_x[2], win.bias_x[3]};
    const f32x4 bias_y = {win.bias_y[0], win.bias_y[1], win.bias_y[2], win.bias_y[3]};
    const EdgeMask edge = make_edge_mask<DT>(kMaskValue * inv_scale, g);     // the model's additive -100, before the scale
    const int strip_tiles = i1 - i0;
#pragma unroll
    for (int jt = 0; jt < (MT + TW - 1) / TW; ++jt) {
        const int li = slot + jt * TW;               // tile inside the strip
        if (li >= strip_tiles) break;
        const int i = i0 + li;
        const int tile_bytes = jt * TW * LL::kTileBytes;         // behind this wave's first tile: a constant
        RowOperand<C> qt;
        read_rows<C>(qt, q_mine + tile_bytes, q_lane);

        // x^T = bias + K . Q^T for the virtual key blocks
        f32x4 s[NBV];
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            RowOperand<C> kop;
            read_rows<C>(kop, k_mine + tile_bytes + vb * LL::kTileBytes, k_lane);
            s[vb] = dot_rows_mma<DT, C>(kop, qt, vb == 1 ? bias_y : bias_x);
        }
        // additive -100 of the model's mask, only on tiles that touch an edge
        const int s0 = 16 * i - shift;           // first row of the window
        const int qrow = 16 * i + n;
        float lse_shift = 0.f;                   // a padded row's logits all carry the -100: its log-sum-exp does too
        if (s0 < 0 || s0 + 16 * NBV > tv) {
            add_edge_mask<DT, NBV>(s, edge, s0 + n, qrow, tv);
            lse_shift = qrow >= tv ? kMaskValue : 0.f;
        }
        float zx[4], zy[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            zx[r] = NBV == 3 ? (win.from0[r] ? s[0][r] : s[NBV - 1][r]) : s[0][r];
            zy[r] = s[1][r];
        }

        const float m = xor_max(max8_of_accumulators(zx, zy));
        const float nm = -m * scale2;

        // The row sums that normalise the output come from the matrix core: a product of the rounded probabilities
        // with a block of ones leaves every lane the sum of its query's row (what the output's numerator was
        // weighted with, so the row is a weighted mean to the last bit), and saves the vector ALU the adds and the
        // cross-lane reduction.  The exact fp32 sum is still formed where the log-sum-exp is asked for, and with
        // dropout, whose row sum is that of the probabilities before any is dropped.
        constexpr bool kMmaSum = !DROP;
        float px[4], py[4], sum = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            px[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(zx[r], scale2, nm));
            py[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(zy[r], scale2, nm));
        }
        if (!kMmaSum || lse) {
#pragma unroll
            for (int r = 0; r < 4; ++r) sum += px[r] + py[r];
            sum = xor_sum(sum);
        }
        if constexpr (DROP) {                    // dropped probabilities leave the sum as it is and O without them
            const uint32_t key = dropout_row_key(dropout_row(drop, b, T, qrow), drop);
            const int j0 = 4 * g - n + L - shift;                    // window slot of register 0 of set X
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int jx = j0 + r + ((NBV == 3 && !win.from0[r]) ? 32 : 0);
                px[r] = dropout_keeps(key, jx, drop) ? px[r] : 0.f;
                py[r] = dropout_keeps(key, j0 + r + 16, drop) ? py[r] : 0.f;
            }
        }
        const u32x2 pkx = {Mma<DT>::pack(px[0], px[1]), Mma<DT>::pack(px[2], px[3])};
        const u32x2 pky = {Mma<DT>::pack(py[0], py[1]), Mma<DT>::pack(py[2], py[3])};

        // O^T = sum over blocks of V_blk^T . P^T
        u32x2 pb[NBV];
        pb[1] = pky;
        if (NBV == 3) {
            pb[0] = u32x2{pkx.x & win.keep0.x, pkx.y & win.keep0.y};
            pb[NBV - 1] = u32x2{pkx.x & win.keep2.x, pkx.y & win.keep2.y};
        } else {
            pb[0] = pkx;
        }
        f32x4 o[CT], rowsum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            LDS_PTR(char) blk = v_mine + tile_bytes + vb * LL::kTileBytes;
            if constexpr (kMmaSum) rowsum = Mma<DT>::k16(ones, pb[vb], rowsum);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) o[ct] = Mma<DT>::k16(read_tr(blk + v_lane.off[ct]), pb[vb], o[ct]);
        }
        const float inv = __builtin_amdgcn_rcpf(kMmaSum ? rowsum[0] : sum) * (DROP ? drop.inv_keep : 1.f);

        // rows past T fall outside the buffer and are dropped by the store
        u32x2 ow[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) ow[ct] = pack_acc<DT>(o[ct], inv);
        const float lse_row = __builtin_fmaf(__builtin_amdgcn_logf(sum) - nm, kLn2, lse_shift);
        if (HG > 1 && out_grouped) {          // into the place of this head's Q tile, which only this wave has read
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
                *reinterpret_cast<LDS_PTR(u32x2)>(q_mine + tile_bytes + LL::addr(n, hw * 2 * C + 32 * ct + 8 * g)) = ow[ct];
        } else {
            store_tile<C>(os, qrow * out_pitch, ow, g, out_whole_lines, out_width);
        }
        if (lse && g == 0) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(lse_row), ls, qrow * 4, 0, 0);
    }
    if (HG > 1 && out_grouped) {
        // The heads of a group lie side by side in the output too: the strip's output rows, collected in the Q
        // region, leave as whole lines - the strip copy run backwards, each lane taking the 16-byte unit that sits
        // at its place in LDS to where it belongs in memory.
        barrier_lds();
        constexpr int kRounds = (region_bytes<CS>(MT) / kChunk + NW - 1) / NW;
        constexpr int kChunkRows = kChunk / LL::kRowBytes;
        const Rsrc gs = make_rsrc(out + sample * outl.sample + head0 * outl.head, min(T, 16 * i1) * outl.pitch);
        const int lane_off = direct_lane_offset<CS>(wave, lane, outl.pitch, HG * outl.width);
        const int chunks = region_bytes<CS>(i1 - i0) / kChunk;
#pragma unroll
        for (int j = 0; j < kRounds; ++j) {
            const int c = j * NW + wave;
            if (c < chunks) {
                const u32x4 unit = *reinterpret_cast<LDS_PTR(u32x4)>(q_lds + c * kChunk + lane * 16);
                __builtin_amdgcn_raw_buffer_store_b128(unit, gs, (16 * i0 + c * kChunkRows) * outl.pitch + lane_off, 0, kStoreAux);
            }
        }
    }
}

// Heads whose rows lie side by side in memory: 16-channel heads four at a time, 32-channel heads two at a time.
inline int head_group(const Geom &g, const Layout &in) {
    const int cw = padded_width(g.C);
    if (cw != g.C || in.head != g.C || cw > 32) return 1;
    const int hg = 64 / cw;
    return (g.H % hg == 0 && in.row >= (int64_t)hg * g.C) ? hg : 1;
}

template <class DT, int C, int HG>
int launch_fwd_hg(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
                  const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &outl, float scale,
                  hipStream_t s) {
    const Split sp = make_split(g.B / HG, g.T, HG > 1 ? kGroupTiles : Strip<C>::kMaxTiles);
    if (!items_ok(sp, g) || !strides_ok(in, g) || !strides_ok(outl, g)) return NA1D_ERR_UNSUPPORTED;
    const bool two = window_blocks(g) == 2;
    // the kernel's form: 0 strips of longer sequences or grouped heads, 1 whole sequences, 2 whole sequences of packed
    // 16-channel rows (where regions for the longest strip cost no workgroup: the forward is not short of LDS there)
    constexpr int kOne = HG == 1 ? 1 : 0, kPacked = HG == 1 && C == 16 ? 2 : kOne;
    const Strides ib = byte_strides(in, g), ob = byte_strides(outl, g);
    auto packed = [&](const Strides &x) {           // [B, T, C] with nothing between rows, heads or samples
        return x.pitch == 2 * C && x.width == 2 * C && x.head == g.T * 2 * C && x.sample == (int64_t)g.H * g.T * 2 * C;
    };
    const int one = HG > 1 || sp.strips != 1 ? 0 : (kPacked == 2 && packed(ib) && packed(ob) && g.T * 2 * C < (1 << 30)) ? 2 : 1;
    auto pick = [&](auto nbv, auto drop) {
        constexpr int N = decltype(nbv)::value;
        constexpr bool D = decltype(drop)::value;
        return one == 2 ? fused_fwd_kernel<DT, C, N, D, HG, kPacked> : one == 1 ? fused_fwd_kernel<DT, C, N, D, HG, kOne>
                                                                                 : fused_fwd_kernel<DT, C, N, D, HG, 0>;
    };
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    auto kern = g.drop.threshold ? (two ? pick(I2{}, std::true_type{}) : pick(I3{}, std::true_type{}))
                                 : (two ? pick(I2{}, std::false_type{}) : pick(I3{}, std::false_type{}));
    const int lt = one == 2 ? Strip<C>::kMaxTiles : sp.nt;          // tiles the regions are laid out for
    const size_t lds = (size_t)2 * region_bytes<C * HG>(lt + 2) + region_bytes<C * HG>(lt) + HG * kBiasEntries * sizeof(float);
    if (!allow_lds(kern, lds)) return NA1D_ERR_LAUNCH;
    note_kernel_as("fused_fwd_kernel<%s, %d, %d, %s, %d, %s>", DT::tag == NA1D_BF16 ? "BF16" : "FP16", C, two ? 2 : 3,
                   g.drop.threshold ? "true" : "false", HG, one == 2 ? "2" : one == 1 ? "1" : "0");
    launch_kernel_block(kern, (unsigned)sp.items, 64u * (HG > 1 ? kGroupWaves : kWaves), lds, s, (char *)out, lse,
                  (const char *)q, (const char *)k, (const char *)v,
                  rpb, t_valid, (uint32_t)sp.items, (int)g.T, g.W, g.L, g.H, sp.tiles, sp.nt, sp.strips, scale,
                  div_magic(sp.strips), div_magic(g.H / HG), byte_strides(in, g), byte_strides(outl, g), window_shift(g),
                  g.drop);
    return launch_status();
}

template <class DT, int C>
int launch_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
               const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &outl, float scale, hipStream_t s) {
    if constexpr (C <= 32) {
        if (head_group(g, in) > 1)
            return launch_fwd_hg<DT, C, 64 / C>(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, s);
    }
    return launch_fwd_hg<DT, C, 1>(out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, s);
}

int fused_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
              const int32_t *t_valid, const Geom &g, const Layout &in, const Layout &outl, float scale, int dtype,
              hipStream_t s) {
    if (!window_blocks(g)) return NA1D_ERR_UNSUPPORTED;
    NA1D_MFMA_DISPATCH(launch_fwd, out, lse, q, k, v, rpb, t_valid, g, in, outl, scale, s);
}

// =============================================================================
// Fused backward
// =============================================================================
// Recomputes P = exp(z - lse) and dP = dO . V^T tile by tile; delta = sum_j P*dP is
// the row sum of the same registers, so O is never read.  Two passes over the
// strip, both entirely out of LDS:
//   pass 1, per query tile (plus one halo tile each side): S^T, dP^T in the
//     "query = lane%16" layout -> P, delta, dS -> dQ^T = K^T . dS^T.  The rounded
//     P and dS tiles stay in registers until every wave is done with K and V.
//   Then they are written over the K/V regions as 16x16 tiles [query][key slot],
//   and pass 2, per key block, reads them back transposed (ds_read_b64_tr_b16) as
//     the B operands of dV^T += dO^T . P and dK^T += Q^T . dS, accumulating in
//     registers over the NBV query tiles that see the block - a gather over the
//     inverse neighbourhood, no atomics, each output row written once, and no
//     second evaluation of the scores.
// d rpb partial sums: one row of kPartialStride floats per work item, folded in a
// fixed order by a second kernel (one workgroup per head).
// Waves per SIMD the register allocation of the backward must leave room for.  16-channel heads: the LDS footprint
// admits six workgroups per CU, so the registers must too (80 or fewer; the dropout variant would spill and is left alone).
constexpr int bwd_min_waves(int C, bool drop, bool one) { return C == 16 && !drop ? (one ? 7 : 6) : 1; }

// Rows that no other workgroup reads: the backward takes them with the workgroup-scope policy rather than the
// non-temporal one of the forward (measured: 4-7 % on the 16-channel backward, nothing either way at 32 channels; the
// forward loses 3-8 % with it).
constexpr int kReadOnceBwd = 1;
constexpr int kBwdMinItems = 256;      // fewer items than this: shorter strips
template <int C> struct StripBwd {
    static constexpr int kMaxTiles = C <= 32 ? 8 : C <= 64 ? 4 : 2;
};
// Floats of the region that first holds the lse of the query-side rows (staged by whole waves, a row per lane) and
// after pass 1 the waves' 32 d rpb slot sums each.
__host__ __device__ inline bool bwd_bias_in_padding(int kv_bytes, int key_region) { return kv_bytes - 2 * key_region >= kBiasEntries * (int)sizeof(float); }
template <int C> constexpr int bwd_lse_rows(bool one) {
    const int rows = ((StripBwd<C>::kMaxTiles + (one ? 0 : 2)) * 16 + 63) / 64 * 64;
    return rows > kWaves * 32 ? rows : kWaves * 32;
}

// ONE: the strip is the whole sequence (strips == 1).  There are no neighbouring strips then and no halo tiles of
// queries either side: two tiles fewer in the Q and dO regions and in a wave's share of pass 1, which is what lets a
// seventh workgroup of 16-channel heads onto a CU (LDS and registers both).
// ONE == 2: such a strip of packed rows as wide as the kernel's C, in and out: the pitch is a constant, the rows of work
// item i start i * T * 2C bytes into every tensor, and the sample / head split waits until the copies are on their way.
template <class DT, int C, int NBV, bool DROP, int ONE>
__global__ void __launch_bounds__(kThreads, bwd_min_waves(C, DROP, ONE != 0))
fused_bwd_kernel(char *__restrict__ dq, char *__restrict__ dk, char *__restrict__ dv, float *__restrict__ drpb,
                 const char *__restrict__ q, const char *__restrict__ k, const char *__restrict__ v,
                 const char *__restrict__ dout, const float *__restrict__ lse, const float *__restrict__ rpb,
                 const int32_t *__restrict__ t_valid, uint32_t items, int T, int W, int L, int H, int tiles, int nt,
                 int strips, float scale, float *__restrict__ drpb_partial, int kv_bytes, uint32_t strips_magic,
                 uint32_t heads_magic, Strides in, Strides outl, int shift_arg, Dropout drop) {
    const int shift = NBV == 3 ? 16 : shift_arg;     // three key blocks always start one tile before the query tile
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    constexpr int MT = StripBwd<C>::kMaxTiles;
    fetch_args_now(dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, items, T, W, L, H, tiles, nt, strips, scale,
                   drpb_partial, kv_bytes, strips_magic, heads_magic, in.sample, in.head, in.pitch, in.width,
                   outl.sample, outl.head, outl.pitch, outl.width, shift_arg);
    if constexpr (DROP) fetch_args_now(drop.threshold, drop.seed_lo, drop.seed_hi, drop.inv_keep, drop.row_stride, drop.row_offset, drop.seq_rows);
    constexpr bool PK = ONE == 2;
    constexpr int HALO = ONE ? 0 : 1;                      // query tiles either side of the strip whose scores pass 2 needs
    constexpr int kRowsQ = (MT + 2 * HALO) * 16;
    constexpr int TPW = (MT + 2 * HALO + kWaves - 1) / kWaves;    // query tiles per wave, at most
    constexpr int kScoreTile = 16 * 16 * 2;                // one 16x16 tile of 16-bit scores
    constexpr int kLseRows = bwd_lse_rows<C>(ONE != 0);
    static_assert(kRowsQ <= kLseRows && kLseRows <= kThreads, "one lane per staged lse row");
    // dynamic LDS (see launch_bwd): [K region | V region] of nt+1+NBV tiles each, starting at the first key of
    // query tile i0-1 (row 16*(i0-1) - shift, so that virtual key blocks are whole tiles of the region), reused after
    // pass 1 for the score tiles and padded to kv_bytes; Q, dO regions of nt + 2*HALO tiles (rows 16*(i0 - HALO) ...); lse
    // of the query-side rows, whose place the 32 d rpb slot sums per wave take after pass 1; the head's bias table
    // where the padding of the K/V regions has no room for it
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int key_region = region_bytes<C>(nt + 1 + NBV), qry_region = region_bytes<C>(nt + 2 * HALO);
    LDS_PTR(char) k_lds = (LDS_PTR(char))smem;
    LDS_PTR(char) v_lds = k_lds + key_region;
    LDS_PTR(char) sc_lds = k_lds;                  // score tiles [(tq*2 + X/Y)*2 + P/dS], tq = query tile - (i0 - HALO)
    LDS_PTR(char) q_lds = k_lds + kv_bytes;
    LDS_PTR(char) g_lds = q_lds + qry_region;      // dO
    LDS_PTR(float) lse_lds = (LDS_PTR(float))(g_lds + qry_region);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // the head's bias table, read before pass 1 only: in what the score tiles need beyond the K and V regions, if that is room enough
    LDS_PTR(float) bias_lds = bwd_bias_in_padding(kv_bytes, key_region) ? (LDS_PTR(float))(k_lds + 2 * key_region) : lse_lds + kLseRows;
    LDS_PTR(float) rsum = lse_lds;                                          // [kWaves][32] d rpb slot sums per wave, once every wave has read its lse
    uint32_t item, sample = 0, head = 0;
    int i0, i1;
    if constexpr (PK) {
        item = blockIdx.x;
        i0 = 0;
        i1 = tiles;
    } else if constexpr (ONE != 0) {   // as in the forward: no strips; packed rows have no neighbours to share an L2 with
        item = in.pitch == 2 * C && outl.pitch == 2 * C ? blockIdx.x : xcd_item(blockIdx.x, items);
        sample = div_by(item, H, heads_magic);
        head = item - sample * H;
        i0 = 0;
        i1 = tiles;
    } else {
        const WorkItem wi = work_item(blockIdx.x, items, strips, strips_magic, H, heads_magic);
        item = wi.item;
        sample = wi.sample;
        head = wi.head;
        i0 = wi.strip * nt;
        i1 = min(i0 + nt, tiles);
    }
    const uint32_t b = ONE ? item : sample * H + head;       // one strip per sequence: the item is the sequence
    const int g = lane >> 4, n = lane & 15;

    const int in_pitch = PK ? 2 * C : in.pitch, out_pitch = PK ? 2 * C : outl.pitch;
    const int in_width = PK ? 2 * C : in.width;
    const int64_t in_off = PK ? (int64_t)((uint64_t)item * (uint32_t)(T * 2 * C)) : sample * in.sample + head * in.head;
    const int64_t out_off = PK ? in_off : sample * outl.sample + head * outl.head;
    {
        const int key_bytes = (ONE ? T : min(T, 16 * (i1 + 2))) * in_pitch;
        const int qry_rows = ONE ? T : min(T, 16 * (i1 + HALO));
        const Rsrc ks = make_rsrc(k + in_off, key_bytes), vs = make_rsrc(v + in_off, key_bytes);
        const Rsrc qs = make_rsrc(q + in_off, qry_rows * in_pitch), gs = make_rsrc(dout + out_off, qry_rows * out_pitch);
        const Rsrc ls = make_rsrc(lse + (int64_t)b * T, T * 4);
        const int lane_off = PK ? direct_lane_offset<C>(wave, lane) : direct_lane_offset<C>(wave, lane, in.pitch, in.width);
        const int lane_off_g = PK ? lane_off : direct_lane_offset<C>(wave, lane, outl.pitch, outl.width);
        // lse of the query-side rows, one per lane (natural log; rows past the region's end are never read)
        if (64 * wave < kRowsQ) load_to_lds<4, 0>(ls, (LDS_PTR(char))(lse_lds + 64 * wave), (16 * (i0 - HALO) + tid) * 4);
        if constexpr (PK) {           // the pitch is the default argument, a constant
            stage_direct<C, MT + 1 + NBV, kReadOnceBwd>(ks, -16 - shift, k_lds, nt + 1 + NBV, wave, lane_off);
            stage_direct<C, MT, kReadOnceBwd>(qs, 0, q_lds, nt, wave, lane_off);
            stage_direct<C, MT + 1 + NBV, kReadOnceBwd>(vs, -16 - shift, v_lds, nt + 1 + NBV, wave, lane_off);
            stage_direct<C, MT, kReadOnceBwd>(gs, 0, g_lds, nt, wave, lane_off);
        } else if (ONE && (in.pitch == 2 * C || C % 64 == 0) && (outl.pitch == 2 * C || C % 64 == 0)) {
            stage_direct<C, MT + 1 + NBV, kReadOnceBwd>(ks, 16 * i0 - 16 - shift, k_lds, nt + 1 + NBV, wave, lane_off, in.pitch);
            stage_direct<C, MT + 2 * HALO, kReadOnceBwd>(qs, 16 * (i0 - HALO), q_lds, nt + 2 * HALO, wave, lane_off, in.pitch);
            stage_direct<C, MT + 1 + NBV, kReadOnceBwd>(vs, 16 * i0 - 16 - shift, v_lds, nt + 1 + NBV, wave, lane_off, in.pitch);
            stage_direct<C, MT + 2 * HALO, kReadOnceBwd>(gs, 16 * (i0 - HALO), g_lds, nt + 2 * HALO, wave, lane_off_g, outl.pitch);
        } else {
            stage_direct<C, MT + 1 + NBV, kReadShared>(ks, 16 * i0 - 16 - shift, k_lds, nt + 1 + NBV, wave, lane_off, in.pitch);
            stage_direct<C, MT + 2 * HALO, kReadShared>(qs, 16 * (i0 - HALO), q_lds, nt + 2 * HALO, wave, lane_off, in.pitch);
            stage_direct<C, MT + 1 + NBV, kReadShared>(vs, 16 * i0 - 16 - shift, v_lds, nt + 1 + NBV, wave, lane_off, in.pitch);
            stage_direct<C, MT + 2 * HALO, kReadShared>(gs, 16 * (i0 - HALO), g_lds, nt + 2 * HALO, wave, lane_off_g, outl.pitch);
        }
    }
    __builtin_amdgcn_sched_barrier(0);       // the copies are on their way: everything else is worked out behind them
    if constexpr (PK) {
        sample = div_by(item, H, heads_magic);
        head = item - sample * H;
    }
    BiasTable bias_raw;                      // (the wait for the copies covers this load too, wherever it is issued)
    load_bias_table(bias_raw, rpb ? rpb + head * W : nullptr, W, lane);

    int tv = T;
    if (t_valid) tv = max(0, min(T, load_uniform_i32(t_valid, sample)));
    // as in the forward: the accumulators start at rpb / scale, z = x * scale * log2(e) - lse is one multiply-add
    const float scale2 = scale * kLog2e;
    const float inv_scale = __builtin_amdgcn_rcpf(scale);

    RowLane<C> key_lane, qry_lane;      // row operands: virtual key block rows / query tile rows
    TrLane<C> key_tr, qry_tr;           // transposed operands of the same
    key_lane.init(0, lane);
    key_tr.init(0, lane);
    qry_lane.init(0, lane);
    qry_tr.init(0, lane);
    // everything that depends on the lane alone is worked out while the copies are in flight
#pragma unroll
    for (int s_ = 0; s_ < (RowOperand<C>::k32 > 0 ? RowOperand<C>::k32 : 1); ++s_) {
        settle(key_lane.off32[s_]);
        settle(qry_lane.off32[s_]);
    }
    settle(key_lane.off16);
    settle(qry_lane.off16);
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        settle(key_tr.off[ct]);
        settle(qry_tr.off[ct]);
    }

    wait_direct();
    wait_bias(bias_raw);
    write_bias_table(bias_lds, bias_raw, W, lane, inv_scale);
    Window<NBV> win;
    read_window<NBV>(win, bias_lds, L, shift, g, n);
    barrier_lds();
    const f32x4 bias_x = {win.bias_x[0], win.bias_x[1], win.bias_x[2], win.bias_x[3]};
    const f32x4 bias_y = {win.bias_y[0], win.bias_y[1], win.bias_y[2], win.bias_y[3]};
    const EdgeMask edge = make_edge_mask<DT>(kMaskValue * inv_scale, g);

    // ---------------- pass 1: query tiles i0-HALO .. i1-1+HALO -> dQ, d rpb, score tiles ----------------
    float racc_x[4] = {0.f, 0.f, 0.f, 0.f}, racc_y[4] = {0.f, 0.f, 0.f, 0.f};
    const Rsrc dqs = make_rsrc(dq + in_off, T * in_pitch);
    const bool dq_whole_lines = stores_whole_lines(in_pitch, C, 0);
    u32x2 sc[TPW][2][2];                // [tile of this wave][X/Y slot set][P / dS], rounded to 16 bit
#pragma unroll
    for (int jt = 0; jt < TPW; ++jt) {
        sc[jt][0][0] = sc[jt][0][1] = sc[jt][1][0] = sc[jt][1][1] = u32x2{0u, 0u};
        const int tq = wave + jt * kWaves;                  // tile index inside the query-side regions
        const int qt = i0 - HALO + tq;
        if (qt >= i1 + HALO || qt < 0 || qt >= tiles) continue;     // nothing there: its scores stay zero
        RowOperand<C> qop, gop;
        read_rows<C>(qop, q_lds + tq * LL::kTileBytes, qry_lane);
        read_rows<C>(gop, g_lds + tq * LL::kTileBytes, qry_lane);
        f32x4 s[NBV], dp[NBV];
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            RowOperand<C> kop, vop;
            const int off = (qt - i0 + 1 + vb) * LL::kTileBytes;
            read_rows<C>(kop, k_lds + off, key_lane);
            read_rows<C>(vop, v_lds + off, key_lane);
            s[vb] = dot_rows_mma<DT, C>(kop, qop, vb == 1 ? bias_y : bias_x);
            dp[vb] = dot_rows_mma<DT, C>(vop, gop);
        }
        float nlse2 = -lse_lds[tq * 16 + n] * kLog2e;
        const int s0 = 16 * qt - shift;
        const int qrow = 16 * qt + n;
        if (s0 < 0 || s0 + 16 * NBV > tv) {
            add_edge_mask<DT, NBV>(s, edge, s0 + n, qrow, tv);
            if (qrow >= tv) nlse2 += kMaskValue * kLog2e;     // a padded row's log-sum-exp carries the -100 its scores do not
        }
        float zx[4], zy[4], dpx[4], dpy[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            zx[r] = NBV == 3 ? (win.from0[r] ? s[0][r] : s[NBV - 1][r]) : s[0][r];
            dpx[r] = NBV == 3 ? (win.from0[r] ? dp[0][r] : dp[NBV - 1][r]) : dp[0][r];
            dpy[r] = dp[1][r];
            zy[r] = s[1][r];
        }
        float px[4], py[4], part = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            px[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(zx[r], scale2, nlse2));
            py[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(zy[r], scale2, nlse2));
        }
        // With dropout mask D (0 or 1/(1-p)): O = (D*P) V, so dV takes D*P and dP = D * (dO . V^T).
        float fx[4] = {1.f, 1.f, 1.f, 1.f}, fy[4] = {1.f, 1.f, 1.f, 1.f};
        if constexpr (DROP) {
            const uint32_t key = dropout_row_key(dropout_row(drop, b, T, qrow), drop);
            const int j0 = 4 * g - n + L - shift;                    // window slot of register 0 of set X
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int jx = j0 + r + ((NBV == 3 && !win.from0[r]) ? 32 : 0);
                fx[r] = dropout_keeps(key, jx, drop) ? drop.inv_keep : 0.f;
                fy[r] = dropout_keeps(key, j0 + r + 16, drop) ? drop.inv_keep : 0.f;
                dpx[r] *= fx[r];
                dpy[r] *= fy[r];
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            part = __builtin_fmaf(px[r], dpx[r], part);
            part = __builtin_fmaf(py[r], dpy[r], part);
        }
        const float delta = xor_sum(part);
        float dsx[4], dsy[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            dsx[r] = px[r] * (dpx[r] - delta);
            dsy[r] = py[r] * (dpy[r] - delta);
            if constexpr (DROP) {      // the probability as the forward used it
                px[r] *= fx[r];
                py[r] *= fy[r];
            }
        }
        sc[jt][0][0] = u32x2{Mma<DT>::pack(px[0], px[1]), Mma<DT>::pack(px[2], px[3])};
        sc[jt][1][0] = u32x2{Mma<DT>::pack(py[0], py[1]), Mma<DT>::pack(py[2], py[3])};
        sc[jt][0][1] = u32x2{Mma<DT>::pack(dsx[0], dsx[1]), Mma<DT>::pack(dsx[2], dsx[3])};
        sc[jt][1][1] = u32x2{Mma<DT>::pack(dsy[0], dsy[1]), Mma<DT>::pack(dsy[2], dsy[3])};
        if (HALO && (qt < i0 || qt >= i1)) continue;        // halo tile: only its scores are needed

#pragma unroll
        for (int r = 0; r < 4; ++r) {
            racc_x[r] += dsx[r];
            racc_y[r] += dsy[r];
        }
        const u32x2 pkx = sc[jt][0][1];
        u32x2 db[NBV];
        db[1] = sc[jt][1][1];
        if (NBV == 3) {
            db[0] = u32x2{pkx.x & win.keep0.x, pkx.y & win.keep0.y};
            db[NBV - 1] = u32x2{pkx.x & win.keep2.x, pkx.y & win.keep2.y};
        } else {
            db[0] = pkx;
        }
        f32x4 acc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            LDS_PTR(char) blk = k_lds + (qt - i0 + 1 + vb) * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) acc[ct] = Mma<DT>::k16(read_tr(blk + key_tr.off[ct]), db[vb], acc[ct]);
        }
        u32x2 qw[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) qw[ct] = pack_acc<DT>(acc[ct], scale);
        store_tile<C>(dqs, qrow * in_pitch, qw, g, dq_whole_lines, in_width);
    }

    // d rpb: the window slot of each of a lane's 8 score registers is the same for every tile, so the lane
    // keeps running sums.  Register r of lane (n, g) holds key a = 4g + r of its block against query n, and the
    // slot depends on a - n only: slot = (a - n + L - shift) mod 32 for set X, 16 more for set Y.  A lane
    // permutation lines the 16 diagonals a - n = d (mod 16) up in lane d; the two members of a class, a - n = d
    // and a - n = d - 16, are told apart by a >= d and go to slots 16 apart, set X and set Y crosswise.  What is
    // left is a sum over the 16 keys a: four registers, then the four lane groups.  Fixed order throughout.
    float s0 = 0.f, s1 = 0.f;             // slots (n + L - shift) mod 32 and 16 further, n = this lane's class
    if (drpb) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int a = 4 * g + r;
            const int from = (16 * g + ((a - n) & 15)) * 4;
            const float x = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(racc_x[r])));
            const float y = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(racc_y[r])));
            const bool upper = a >= n;     // a - n = d, else d - 16
            s0 += upper ? x : y;
            s1 += upper ? y : x;
        }
        s0 = xor_sum(s0);
        s1 = xor_sum(s1);
    }

    barrier_lds();                    // every wave is done with K, V and lse: their regions become the score tiles and the d rpb sums
    if (drpb) {
        const int slot = (n + L - shift) & 31;
        if (g == 0) rsum[wave * 32 + slot] = s0;
        if (g == 1) rsum[wave * 32 + ((slot + 16) & 31)] = s1;
    }
#pragma unroll
    for (int jt = 0; jt < TPW; ++jt) {
        const int tq = wave + jt * kWaves;
        const int qt = i0 - HALO + tq;
        if (qt >= i1 + HALO || qt < 0 || qt >= tiles) continue;              // no such tile: pass 2 does not look for it
        LDS_PTR(char) t = sc_lds + tq * 4 * kScoreTile + n * 32 + g * 8;   // tile[query n][key slots 4g..4g+3]
#pragma unroll
        for (int xy = 0; xy < 2; ++xy)
#pragma unroll
            for (int pd = 0; pd < 2; ++pd) *reinterpret_cast<LDS_PTR(u32x2)>(t + (xy * 2 + pd) * kScoreTile) = sc[jt][xy][pd];
    }
    barrier_lds();

    // ---------------- pass 2: key blocks of the strip -> dK, dV ----------------
    // key block kp covers rows 16*kp - shift .. +15 and is virtual block vb of query tile kp - vb.  Lane (n, g)
    // of the transposed score read holds tile[query 4g+r][key slot n]; in a merged tile that entry belongs to
    // block 0 when n - (4g+r) - shift + L >= 0 and to block 2 otherwise.
    u32x2 keep0t = {0xffffffffu, 0xffffffffu};
    if (NBV == 3) {
        uint32_t m[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) m[r] = (n - (4 * g + r) - shift + L >= 0) ? 0xffffu : 0u;
        keep0t = u32x2{m[0] | (m[1] << 16), m[2] | (m[3] << 16)};
    }
    const int sc_lane = (4 * g + (n >> 2)) * 32 + (n & 3) * 8;       // transposed read of a score tile
    const int row_lo = 16 * i0, row_hi = min(T, 16 * i1);            // rows this strip owns
    const Rsrc dks = make_rsrc(dk + in_off + (int64_t)row_lo * in_pitch, (row_hi - row_lo) * in_pitch);
    const Rsrc dvs = make_rsrc(dv + in_off + (int64_t)row_lo * in_pitch, (row_hi - row_lo) * in_pitch);
    const int kp_lo = i0 + (shift == 16 ? 1 : 0), kp_hi = i1 - (shift == 0 ? 1 : 0);
    // a key block starts `shift` rows before a tile (non-temporal stores of split lines cost cfg2's backward 5 %;
    // where lines are whole they gain 10 %)
    const bool whole_lines = stores_whole_lines(in_pitch, C, shift);
    for (int kp = kp_lo + wave; kp <= kp_hi; kp += kWaves) {
        f32x4 acck[CT], accv[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acck[ct] = accv[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            // a query tile outside the sequence (its Q and dO rows were staged as zeros) has no score tile: read one
            // that is there and drop what it holds
            const bool there = (uint32_t)(kp - vb) < (uint32_t)tiles;
            const uint32_t tm = there ? 0xffffffffu : 0u;
            const int tq = there ? kp - vb - (i0 - HALO) : HALO;       // a tile that is there, whatever it holds
            LDS_PTR(char) qtile = q_lds + tq * LL::kTileBytes;
            LDS_PTR(char) gtile = g_lds + tq * LL::kTileBytes;
            LDS_PTR(char) stile = sc_lds + (tq * 4 + (vb == 1 ? 2 : 0)) * kScoreTile + sc_lane;
            u32x2 pb = read_tr(stile), db = read_tr(stile + kScoreTile);
            if (NBV == 3 && vb == 0) {
                pb = u32x2{pb.x & keep0t.x & tm, pb.y & keep0t.y & tm};
                db = u32x2{db.x & keep0t.x & tm, db.y & keep0t.y & tm};
            } else if (NBV == 3 && vb == 2) {
                pb = u32x2{pb.x & ~keep0t.x & tm, pb.y & ~keep0t.y & tm};
                db = u32x2{db.x & ~keep0t.x & tm, db.y & ~keep0t.y & tm};
            } else {
                pb = u32x2{pb.x & tm, pb.y & tm};
                db = u32x2{db.x & tm, db.y & tm};
            }
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                accv[ct] = Mma<DT>::k16(read_tr(gtile + qry_tr.off[ct]), pb, accv[ct]);
                acck[ct] = Mma<DT>::k16(read_tr(qtile + qry_tr.off[ct]), db, acck[ct]);
            }
        }
        const int row_off = (16 * (kp - i0) - shift + n) * in_pitch;    // outside the strip -> dropped
        u32x2 kw[CT], vw[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            kw[ct] = pack_acc<DT>(acck[ct], scale);
            vw[ct] = pack_acc<DT>(accv[ct], 1.f);
        }
        store_tile<C>(dks, row_off, kw, g, whole_lines, in_width);
        store_tile<C>(dvs, row_off, vw, g, whole_lines, in_width);
    }

    // last, behind the gradient stores: issued earlier (the sums are complete before pass 2) the atomics cost the
    // kernel twice as much, the stores of pass 2 queueing behind them
    if (drpb && tid < W) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) t += rsum[w * 32 + tid];
        if (drpb_partial)
            drpb_partial[(size_t)item * kPartialStride + tid] = t;   // folded by drpb_reduce_kernel
        else
            atomicAdd(drpb + head * W + tid, t);
    }
}

template <class DT, int C>
int launch_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
               const void *dout, const float *lse, const float *rpb, const int32_t *t_valid, const Geom &g,
               const Layout &in, const Layout &outl, float scale, float *workspace, int64_t workspace_bytes,
               hipStream_t s) {
    const Split sp = make_split(g.B, g.T, StripBwd<C>::kMaxTiles, kBwdMinItems);
    if (!items_ok(sp, g) || !strides_ok(in, g) || !strides_ok(outl, g)) return NA1D_ERR_UNSUPPORTED;
    // a workspace that is passed is used or refused: falling back to atomics would silently give up the fixed order
    // the caller asked for
    float *partial = nullptr;
    if (drpb && workspace) {
        if (workspace_bytes < sp.items * kPartialStride * (int64_t)sizeof(float)) return NA1D_ERR_WORKSPACE;
        partial = workspace;
    }
    const bool two = window_blocks(g) == 2;
    const bool one = sp.strips == 1;
    const Strides ib = byte_strides(in, g), ob = byte_strides(outl, g);
    auto packed = [&](const Strides &x) {           // [B, T, C] with nothing between rows, heads or samples
        return x.pitch == 2 * C && x.width == 2 * C && x.head == g.T * 2 * C && x.sample == (int64_t)g.H * g.T * 2 * C;
    };
    const int form = !one ? 0 : packed(ib) && packed(ob) && g.T * 2 * C < (1 << 30) ? 2 : 1;      // see the kernel's ONE
    auto pick = [&](auto nbv, auto drop) {
        constexpr int N = decltype(nbv)::value;
        constexpr bool D = decltype(drop)::value;
        return form == 2 ? fused_bwd_kernel<DT, C, N, D, 2> : form == 1 ? fused_bwd_kernel<DT, C, N, D, 1> : fused_bwd_kernel<DT, C, N, D, 0>;
    };
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    auto kern = g.drop.threshold ? (two ? pick(I2{}, std::true_type{}) : pick(I3{}, std::true_type{}))
                                 : (two ? pick(I2{}, std::false_type{}) : pick(I3{}, std::false_type{}));
    // the K and V regions double as the score tiles of pass 2 (4 tiles of 512 B per query tile)
    // (a strip that is the whole sequence has no halo tiles)
    const int halo = one ? 0 : 1;
    const int kv_bytes = std::max(2 * region_bytes<C>(sp.nt + 1 + window_blocks(g)), (sp.nt + 2 * halo) * 4 * 512);
    const bool bias_apart = !bwd_bias_in_padding(kv_bytes, region_bytes<C>(sp.nt + 1 + window_blocks(g)));
    const size_t lds = (size_t)kv_bytes + (size_t)2 * region_bytes<C>(sp.nt + 2 * halo) +
                       (bwd_lse_rows<C>(one) + (bias_apart ? kBiasEntries : 0)) * sizeof(float);
    if (!allow_lds(kern, lds)) return NA1D_ERR_LAUNCH;
    note_kernel_as("fused_bwd_kernel<%s, %d, %d, %s, %s>", DT::tag == NA1D_BF16 ? "BF16" : "FP16", C, two ? 2 : 3,
                   g.drop.threshold ? "true" : "false", form == 2 ? "2" : form == 1 ? "1" : "0");
    launch_kernel(kern, (unsigned)sp.items, lds, s, (char *)dq, (char *)dk, (char *)dv, drpb, (const char *)q,
                  (const char *)k, (const char *)v, (const char *)dout, lse, rpb, t_valid, (uint32_t)sp.items, (int)g.T,
                  g.W, g.L, g.H, sp.tiles, sp.nt, sp.strips, scale, partial, kv_bytes, div_magic(sp.strips),
                  div_magic(g.H), ib, ob, window_shift(g), g.drop);
    // not behind a launch that was refused (events set on a capturing stream): the sums it would fold do not exist
    if (partial && drpb && !launch_events().refused)
        drpb_reduce_kernel<kPartialStride><<<(unsigned)(g.H * g.W), 128, 0, s>>>(drpb, partial, (int)(g.B / g.H), g.H, sp.strips, g.W);
    return launch_status();
}

template <class DT, int C>
int64_t bwd_workspace(const Geom &g) {
    return make_split(g.B, g.T, StripBwd<C>::kMaxTiles, kBwdMinItems).items * kPartialStride * (int64_t)sizeof(float);
}

int fused_bwd(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
              const void *out, const void *dout, const float *lse, const float *rpb, const int32_t *t_valid,
              const Geom &g, const Layout &in, const Layout &outl, float scale, int dtype, float *workspace,
              int64_t workspace_bytes, hipStream_t s) {
    (void)out;   // delta is recomputed from P and dP; O is not needed
    if (!window_blocks(g)) return NA1D_ERR_UNSUPPORTED;
    NA1D_MFMA_DISPATCH(launch_bwd, dq, dk, dv, drpb, q, k, v, dout, lse, rpb, t_valid, g, in, outl, scale, workspace,
                       workspace_bytes, s);
}

int64_t fused_bwd_workspace_bytes(const Geom &g, int dtype) {
    if (!window_blocks(g)) return wide_bwd_workspace_bytes(g);     // 0 where the wide kernels do not cover the shape either
    switch (padded_width(g.C)) {   // the split does not depend on the dtype
        case 16: return bwd_workspace<BF16, 16>(g);
        case 32: return bwd_workspace<BF16, 32>(g);
        case 64: return bwd_workspace<BF16, 64>(g);
        case 128: return bwd_workspace<BF16, 128>(g);
    }
    (void)dtype;
    return 0;
}

// ---- scratch of the entry point that allocates nothing -----------------------------------------------------
// na1d_fused_backward_noalloc() keeps the d rpb partial sums (one row of kPartialStride floats per workgroup) in
// this array instead of a caller's workspace.  Every GPU the library runs on holds its own copy at its own
// address until the process ends.  In host code the name `scratch` is only a handle: the device address comes
// from hipGetSymbolAddress, once per device with that device current, and that pointer is what kernels get.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

int static_scratch(float **ptr) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void *per_device[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return NA1D_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return NA1D_ERR_LAUNCH;
        }
        per_device[dev] = p;
    }
    *ptr = static_cast<float *>(per_device[dev]);
    return NA1D_OK;
}

}  // namespace mfma
}  // namespace na1d
