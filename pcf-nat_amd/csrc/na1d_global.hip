// Dense ("global") attention of the models' two global layers on the matrix cores (gfx950):
//   P = softmax(q k^T * scale + M),  O = P v,   M[t, u] = -100 where row t or column u is padded
// (models/PCF_NATransformer.py:199-221 with the mask of :406-414).  Flash-attention style, built
// from the tile machinery of na1d_mfma_core.h: S^T tiles of 16 keys x 16 queries, an online
// softmax whose row statistics are lane-local up to a reduction over the four lane groups, and
// the rounded probabilities fed straight back as the B operand of O^T += V^T P^T.
//
// Sequences of up to 128 rows (the models run at about 100): one workgroup per sequence with everything it needs whole
// in LDS behind one barrier - a forward with a plain softmax, and a backward that is ONE kernel (delta never leaves the
// chip, every input is read once).
// Longer sequences: the forward owns 4 or 8 query tiles per workgroup (one or two per wave) and walks the keys in
// chunks of 4 tiles that all four waves share through LDS, the next chunk in flight behind the current one.
// Their backward: one kernel per query strip computes delta = rowsum(dO * O) and dQ, walking the keys;
// a second per key strip computes dK and dV, walking the queries with Q and K swapped in the
// score product so that the probabilities come out as "lane = key, registers = queries", which
// is the B operand of dV^T += dO^T P and dK^T += Q^T dS.  No atomics, every output written once.
#include <type_traits>

#include "na1d_mfma_core.h"

namespace na1d {
namespace mfma {

constexpr int kStripTiles = 4;      // tiles per strip (one per wave) and per chunk
static_assert(kStripTiles == kWaves, "one tile of the strip per wave");

// Two 16-bit values of a register as floats.
template <class DT> __device__ inline f32x2 unpack2(uint32_t w);
template <> __device__ inline f32x2 unpack2<BF16>(uint32_t w) {
    return f32x2{__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u)};
}
template <> __device__ inline f32x2 unpack2<FP16>(uint32_t w) {
    return __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
}
// sum over this lane's channels of a[c] * b[c] for two row operands
template <class DT, int C>
__device__ inline float dot_lane(const RowOperand<C> &a, const RowOperand<C> &b) {
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < RowOperand<C>::k32; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f32x2 x = unpack2<DT>(a.w32[s][i]), y = unpack2<DT>(b.w32[s][i]);
            acc = __builtin_fmaf(x.x, y.x, __builtin_fmaf(x.y, y.y, acc));
        }
    if (RowOperand<C>::k16)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const f32x2 x = unpack2<DT>(a.w16[0][i]), y = unpack2<DT>(b.w16[0][i]);
            acc = __builtin_fmaf(x.x, y.x, __builtin_fmaf(x.y, y.y, acc));
        }
    return acc;
}

// x *= a in the registers x lives in.  Written as plain C++ inside a branch, the compiler gives the products new
// registers and pays for it with copies of every accumulator on both sides of the branch.  The accumulators are
// results of matrix instructions the compiler cannot relate to this block: callers keep at least a dozen
// instructions between the last of those and this.  The factor may come straight out of a transcendental
// instruction, whose result an ordinary vector instruction may read one state later at the earliest: hence the s_nop.
__device__ inline void scale_in_place(f32x4 &x, float a) {
    asm volatile("s_nop 0\n\tv_mul_f32 %0, %4, %0\n\tv_mul_f32 %1, %4, %1\n\tv_mul_f32 %2, %4, %2\n\tv_mul_f32 %3, %4, %3"
                 : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3])
                 : "v"(a));
}

struct GlobalArgs {
    int T, H, strips;            // strips of kStripTiles tiles per sequence
    uint32_t strips_magic, heads_magic;
    int pitch;                   // bytes per row = 2 * head_dim (packed rows)
    float scale;
    Dropout drop;                // attention dropout; its window slot is the key's row index
};

// =============================================================================
// Forward
// =============================================================================
// A workgroup owns 4 * QT query tiles, QT to a wave (tiles wave, wave + 4, ...), and walks the keys in chunks of 4
// tiles that all waves share through LDS; the next chunk is on its way while this one is worked on, so one barrier a
// chunk.  The wave's query tiles go from memory straight into the registers of the matrix operand.
//
// The softmax costs more vector instructions than the two products cost matrix instructions, so a chunk whose keys
// all count takes a short form: the running maximum comes from the raw products (the scale is positive) and scale
// and maximum fold into one multiply-add in front of the exponential.  Chunks that reach past the valid keys take the long form with its masks.  A padded
// query row has -100 added to every score: a constant that leaves its probabilities alone and moves its LSE, which
// is where it is added.
template <class DT, int C, bool DROP, int QT>
__global__ void __launch_bounds__(kThreads)
global_fwd_kernel(char *__restrict__ out, float *__restrict__ lse, const char *__restrict__ q,
                  const char *__restrict__ k, const char *__restrict__ v, const int32_t *__restrict__ t_valid,
                  uint32_t items, GlobalArgs a) {
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    fetch_args_now(out, lse, q, k, v, t_valid, items, a.T, a.H, a.strips, a.strips_magic, a.heads_magic, a.pitch, a.scale);
    if constexpr (DROP) fetch_args_now(a.drop.threshold, a.drop.seed_lo, a.drop.seed_hi, a.drop.inv_keep);
    constexpr int kStep = region_bytes<C>(kStripTiles);
    extern __shared__ __attribute__((aligned(16))) char smem[];          // 4 * kStep bytes: K and V of two chunks
    LDS_PTR(char) kv_lds = (LDS_PTR(char))smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, n = lane & 15;
    const uint32_t item = xcd_item(blockIdx.x, items);
    const uint32_t b = div_by(item, a.strips, a.strips_magic);
    const int strip = (int)(item - b * a.strips);
    const uint32_t sample = div_by(b, a.H, a.heads_magic);
    const int T = a.T, tiles = (T + 15) >> 4;

    const int64_t seq_off = (int64_t)b * T * a.pitch;
    const Rsrc qs = make_rsrc(q + seq_off, T * a.pitch), ks = make_rsrc(k + seq_off, T * a.pitch);
    const Rsrc vs = make_rsrc(v + seq_off, T * a.pitch), os = make_rsrc(out + seq_off, T * a.pitch);
    const Rsrc ls = make_rsrc(lse ? lse + (int64_t)b * T : nullptr, lse ? T * 4 : 0);
    const int lane_off = direct_lane_offset<C>(wave, lane, a.pitch, a.pitch);
    stage_direct<C, kStripTiles, kReadShared>(ks, 0, kv_lds, kStripTiles, wave, lane_off, a.pitch);
    stage_direct<C, kStripTiles, kReadShared>(vs, 0, kv_lds + kStep, kStripTiles, wave, lane_off, a.pitch);
    int qt[QT];                                             // this wave's query tiles
    RowOperand<C> qop[QT];
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        qt[h] = kStripTiles * (QT * strip + h) + wave;
        load_rows<C, kReadShared>(qop[h], qs, 16 * qt[h] * a.pitch, a.pitch, a.pitch, lane);
    }
    int tv = T;
    if (t_valid) tv = max(0, min(T, t_valid[sample]));
    const float scale2 = a.scale * kLog2e, mask2 = kMaskValue * kLog2e;     // the scale is positive: checked at the C boundary

    RowLane<C> row_lane;
    TrLane<C> tr_lane;
    row_lane.init(0, lane);
    tr_lane.init(0, lane);
    constexpr float kSlack = 6.f;
    float m[QT], l[QT];
    f32x4 o[QT][CT], lsum[QT];                              // lsum: the row sum in every register, without dropout
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        m[h] = kNegInf;
        l[h] = 0.f;
        lsum[h] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[h][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // one chunk of keys; `whole`: all of its 64 keys exist and count
    auto chunk = [&](auto whole, int c0, LDS_PTR(char) k_lds, LDS_PTR(char) v_lds) {
        constexpr bool kWhole = decltype(whole)::value;
        const int nk = kWhole ? kStripTiles : min(kStripTiles, tiles - c0);      // key tiles in this chunk
        f32x4 s[QT][kStripTiles];
#pragma unroll
        for (int kt = 0; kt < kStripTiles; ++kt) {
            if (kt < nk) {
                RowOperand<C> kop;
                read_rows<C>(kop, k_lds + kt * LL::kTileBytes, row_lane);
#pragma unroll
                for (int h = 0; h < QT; ++h) s[h][kt] = dot_rows_mma<DT, C>(kop, qop[h]);
            }
        }
        u32x4 pp[QT][kStripTiles / 2];          // probabilities of two key tiles: the B operand of a 32-deep product
#pragma unroll
        for (int h = 0; h < QT; ++h) {
            const int qrow = 16 * qt[h] + n;
            const uint32_t drop_key = DROP ? dropout_row_key((uint64_t)b * T + qrow, a.drop) : 0u;
            float mc = kNegInf;
            if constexpr (kWhole) {
#pragma unroll
                for (int kt = 0; kt < kStripTiles; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) mc = __builtin_fmaxf(mc, s[h][kt][r]);
                mc = xor_max(mc) * scale2;
            } else {
                const bool row_masked = qrow >= tv;
#pragma unroll
                for (int kt = 0; kt < kStripTiles; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = 16 * (c0 + kt) + 4 * g + r;
                        const float zz = s[h][kt][r] * scale2 + ((key >= tv && !row_masked) ? mask2 : 0.f);
                        s[h][kt][r] = kt < nk && key < T ? zz : kNegInf;      // rows past the sequence do not exist
                        mc = __builtin_fmaxf(mc, s[h][kt][r]);
                    }
                mc = xor_max(mc);                           // finite: key 16 * c0 exists
            }
            // The reference point of the exponentials moves only when a row's maximum has outgrown it by more than
            // kSlack (probabilities then stay below 2^kSlack, which every format here holds): most chunks leave
            // the accumulators as they are.
            if (__builtin_amdgcn_ballot_w64(mc > m[h] + kSlack)) {
                const float m_new = max2(m[h], mc);
                const float alpha = __builtin_amdgcn_exp2f(m[h] - m_new);
                m[h] = m_new;
                l[h] *= alpha;
                if constexpr (!DROP) scale_in_place(lsum[h], alpha);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) scale_in_place(o[h][ct], alpha);
            }
            const float ref = -m[h];
            float part = 0.f;
#pragma unroll
            for (int kt = 0; kt < kStripTiles; ++kt) {
                float p[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    p[r] = __builtin_amdgcn_exp2f(kWhole ? __builtin_fmaf(s[h][kt][r], scale2, ref) : s[h][kt][r] + ref);
                    if constexpr (DROP) {                   // a dropped probability stays in the sum and leaves O
                        part += p[r];
                        if (!dropout_keeps(drop_key, 16 * (c0 + kt) + 4 * g + r, a.drop)) p[r] = 0.f;
                    }
                }
                pp[h][kt / 2][2 * (kt & 1)] = Mma<DT>::pack(p[0], p[1]);
                pp[h][kt / 2][2 * (kt & 1) + 1] = Mma<DT>::pack(p[2], p[3]);
            }
            if constexpr (DROP) l[h] += xor_sum(part);
        }
        // O^T += V^T P^T over two key tiles at a time (the 32-deep product costs what the 16-deep one does); a tile
        // past the chunk's last has zero probabilities and zeros in LDS.  Without dropout the row sums come from
        // the same instruction with ones in place of V^T.
#pragma unroll
        for (int kt = 0; kt < kStripTiles; kt += 2) {
            if (kt >= nk) continue;
            LDS_PTR(char) blk = v_lds + kt * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const u32x2 v0 = read_tr(blk + tr_lane.off[ct]), v1 = read_tr(blk + LL::kTileBytes + tr_lane.off[ct]);
                const u32x4 vv = {v0.x, v0.y, v1.x, v1.y};
#pragma unroll
                for (int h = 0; h < QT; ++h) o[h][ct] = Mma<DT>::k32(vv, pp[h][kt / 2], o[h][ct]);
            }
            if constexpr (!DROP) {
                const uint32_t one = Mma<DT>::pack(1.f, 1.f);
                const u32x4 ones = {one, one, one, one};
#pragma unroll
                for (int h = 0; h < QT; ++h) lsum[h] = Mma<DT>::k32(ones, pp[h][kt / 2], lsum[h]);
            }
        }
    };

    // Chunks whose keys all count come first and have a loop of their own: with both forms in one loop body the
    // accumulators change registers where the two meet, at the price of a copy of each per chunk.
    const int whole_keys = min(T, tv);
    int at = 0;                                             // byte offset of the chunk's pair of regions: 0 or 2 * kStep
    auto step = [&](auto whole, int c0) {
        wait_direct();
        barrier_lds();      // this chunk has landed, and every wave is done with the one before, whose regions the next takes
        if (c0 + kStripTiles < tiles) {
            LDS_PTR(char) next = kv_lds + (at ^ 2 * kStep);
            stage_direct<C, kStripTiles, kReadShared>(ks, 16 * (c0 + kStripTiles), next, kStripTiles, wave, lane_off, a.pitch);
            stage_direct<C, kStripTiles, kReadShared>(vs, 16 * (c0 + kStripTiles), next + kStep, kStripTiles, wave, lane_off, a.pitch);
        }
        chunk(whole, c0, kv_lds + at, kv_lds + at + kStep);
        at ^= 2 * kStep;
    };
    int c0 = 0;
    for (; 16 * (c0 + kStripTiles) <= whole_keys; c0 += kStripTiles) step(std::true_type{}, c0);
    for (; c0 < tiles; c0 += kStripTiles) step(std::false_type{}, c0);
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        if (qt[h] >= tiles) break;
        const int qrow = 16 * qt[h] + n;
        if constexpr (!DROP) l[h] = lsum[h][0];
        const float inv = __builtin_amdgcn_rcpf(l[h]) * (DROP ? a.drop.inv_keep : 1.f);
        u32x2 ow[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) ow[ct] = pack_acc<DT>(o[h][ct], inv);
        store_tile<C>(os, qrow * a.pitch, ow, g, stores_whole_lines(a.pitch, C, 0), a.pitch);   // rows past T are dropped
        const float pad = qrow >= tv ? kMaskValue : 0.f;
        if (g == 0)
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint((m[h] + __builtin_amdgcn_logf(l[h])) * kLn2 + pad), ls, qrow * 4, 0, 0);
    }
}

// =============================================================================
// Forward for sequences of up to 128 rows (the models' dense layers run at about 100): one workgroup per sequence,
// keys and values whole in LDS behind a single barrier, every wave two query tiles (wave and wave + 4) that share each
// key and value operand it reads.  All scores of a row are in registers at once, so the softmax is a plain one.
// =============================================================================
constexpr int kShortTiles = 8;      // longest sequence of the short forms, in tiles
template <class DT, int C, bool DROP, int TILES, int QT>
__global__ void __launch_bounds__(64 * TILES / QT)
global_fwd_short_kernel(char *__restrict__ out, float *__restrict__ lse, const char *__restrict__ q,
                        const char *__restrict__ k, const char *__restrict__ v, const int32_t *__restrict__ t_valid,
                        GlobalArgs a) {
    using LL = Lds<C>;
    constexpr int CT = C / 16, kW = TILES / QT;       // waves of the workgroup, QT query tiles each
    fetch_args_now(out, lse, q, k, v, t_valid, a.T, a.H, a.heads_magic, a.pitch, a.scale);
    if constexpr (DROP) fetch_args_now(a.drop.threshold, a.drop.seed_lo, a.drop.seed_hi, a.drop.inv_keep);
    const int T = a.T, tiles = (T + 15) >> 4, pitch = a.pitch;      // rows of head_dim channels, zero-padded to C on the way in
    extern __shared__ __attribute__((aligned(16))) char smem[];          // 2 * region_bytes<C>(tiles)
    LDS_PTR(char) k_lds = (LDS_PTR(char))smem;
    LDS_PTR(char) v_lds = k_lds + region_bytes<C>(tiles);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, n = lane & 15;
    const uint32_t b = blockIdx.x;
    const int64_t seq_off = (int64_t)((uint64_t)b * (uint32_t)(T * pitch));
    const Rsrc ks = make_rsrc(k + seq_off, T * pitch), vs = make_rsrc(v + seq_off, T * pitch);
    const Rsrc qs = make_rsrc(q + seq_off, T * pitch);
    const int lane_off = direct_lane_offset<C>(wave, lane, pitch, pitch);
    stage_direct<C, TILES, kReadOnce, kW>(ks, 0, k_lds, tiles, wave, lane_off, pitch);
    stage_direct<C, TILES, kReadOnce, kW>(vs, 0, v_lds, tiles, wave, lane_off, pitch);
    RowOperand<C> qop[QT];
#pragma unroll
    for (int h = 0; h < QT; ++h) load_rows<C, kReadOnce>(qop[h], qs, 16 * (wave + kW * h) * pitch, pitch, pitch, lane);
    __builtin_amdgcn_sched_barrier(0);

    const uint32_t sample = div_by(b, a.H, a.heads_magic);
    int tv = T;
    if (t_valid) tv = max(0, min(T, t_valid[sample]));
    const Rsrc os = make_rsrc(out + seq_off, T * pitch);
    const Rsrc ls = make_rsrc(lse ? lse + (int64_t)b * T : nullptr, lse ? T * 4 : 0);
    const float scale2 = a.scale * kLog2e, mask2 = kMaskValue * kLog2e;
    RowLane<C> row_lane;
    TrLane<C> tr_lane;
    row_lane.init(0, lane);
    tr_lane.init(0, lane);
    wait_direct();
    barrier_lds();

    // Scores of all keys, in the log2 domain.  A tile whose 16 keys all count needs the scale only; a padded query
    // row has -100 added to every score, which leaves its probabilities alone and moves its LSE: added there.
    const int whole_keys = min(T, tv);
    float z[QT][TILES][4];
#pragma unroll
    for (int kt = 0; kt < TILES; ++kt) {
        if (kt < tiles) {
            RowOperand<C> kop;
            read_rows<C>(kop, k_lds + kt * LL::kTileBytes, row_lane);
            f32x4 s[QT];
#pragma unroll
            for (int h = 0; h < QT; ++h) s[h] = dot_rows_mma<DT, C>(kop, qop[h]);
            if (16 * (kt + 1) <= whole_keys) {
#pragma unroll
                for (int h = 0; h < QT; ++h)
#pragma unroll
                    for (int r = 0; r < 4; ++r) z[h][kt][r] = s[h][r] * scale2;
            } else {
#pragma unroll
                for (int h = 0; h < QT; ++h) {
                    const bool row_masked = 16 * (wave + kW * h) + n >= tv;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = 16 * kt + 4 * g + r;
                        const float zz = s[h][r] * scale2 + ((key >= tv && !row_masked) ? mask2 : 0.f);
                        z[h][kt][r] = key < T ? zz : kNegInf;   // rows past the sequence do not exist
                    }
                }
            }
        } else {
#pragma unroll
            for (int h = 0; h < QT; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) z[h][kt][r] = kNegInf;
        }
        // left alone, the scheduler reads every key tile before the first product and runs out of registers
        if (kt & 1) __builtin_amdgcn_sched_barrier(0);
    }
    u32x2 pb[QT][TILES];
    float m[QT], l[QT];
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        const int qrow = 16 * (wave + kW * h) + n;
        float mc = kNegInf;
#pragma unroll
        for (int kt = 0; kt < TILES; ++kt) mc = max3(mc, max2(z[h][kt][0], z[h][kt][1]), max2(z[h][kt][2], z[h][kt][3]));
        m[h] = xor_max(mc);                                 // finite: key 0 exists
        const uint32_t drop_key = DROP ? dropout_row_key((uint64_t)b * T + qrow, a.drop) : 0u;
        float part = 0.f;
#pragma unroll
        for (int kt = 0; kt < TILES; ++kt) {
            if (kt < tiles) {
                float p[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    p[r] = __builtin_amdgcn_exp2f(z[h][kt][r] - m[h]);
                    if constexpr (DROP) {                   // a dropped probability stays in the sum and leaves O
                        part += p[r];
                        if (!dropout_keeps(drop_key, 16 * kt + 4 * g + r, a.drop)) p[r] = 0.f;
                    }
                }
                pb[h][kt] = u32x2{Mma<DT>::pack(p[0], p[1]), Mma<DT>::pack(p[2], p[3])};
            } else {
                pb[h][kt] = u32x2{0u, 0u};
            }
        }
        l[h] = DROP ? xor_sum(part) : 0.f;
    }
    // O^T = V^T P^T, two key tiles to a 32-deep product.  Without dropout the row sums come from the same instruction
    // with ones in place of V^T.  An accumulator sees products of one depth only: a 16-deep product that takes the
    // result of a 32-deep one as its accumulator straight behind it has read stale values here.
    f32x4 o[QT][CT], lsum[QT];
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        lsum[h] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[h][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const uint32_t one = Mma<DT>::pack(1.f, 1.f);
#pragma unroll
    for (int kt = 0; kt < TILES; kt += 2) {
        if (kt >= tiles) continue;
        LDS_PTR(char) blk = v_lds + kt * LL::kTileBytes;
        if (kt + 1 < tiles) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const u32x2 v0 = read_tr(blk + tr_lane.off[ct]), v1 = read_tr(blk + LL::kTileBytes + tr_lane.off[ct]);
                const u32x4 vv = {v0.x, v0.y, v1.x, v1.y};
#pragma unroll
                for (int h = 0; h < QT; ++h)
                    o[h][ct] = Mma<DT>::k32(vv, u32x4{pb[h][kt].x, pb[h][kt].y, pb[h][kt + 1].x, pb[h][kt + 1].y}, o[h][ct]);
            }
            if constexpr (!DROP)
#pragma unroll
                for (int h = 0; h < QT; ++h)
                    lsum[h] = Mma<DT>::k32(u32x4{one, one, one, one},
                                           u32x4{pb[h][kt].x, pb[h][kt].y, pb[h][kt + 1].x, pb[h][kt + 1].y}, lsum[h]);
        } else {                // a last single tile against zeros in the other half: one kind of product per accumulator
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const u32x2 vt = read_tr(blk + tr_lane.off[ct]);
#pragma unroll
                for (int h = 0; h < QT; ++h)
                    o[h][ct] = Mma<DT>::k32(u32x4{vt.x, vt.y, 0u, 0u}, u32x4{pb[h][kt].x, pb[h][kt].y, 0u, 0u}, o[h][ct]);
            }
            if constexpr (!DROP)
#pragma unroll
                for (int h = 0; h < QT; ++h)
                    lsum[h] = Mma<DT>::k32(u32x4{one, one, 0u, 0u}, u32x4{pb[h][kt].x, pb[h][kt].y, 0u, 0u}, lsum[h]);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        if (wave + kW * h >= tiles) break;
        const int qrow = 16 * (wave + kW * h) + n;
        if constexpr (!DROP) l[h] = lsum[h][0];
        const float inv = __builtin_amdgcn_rcpf(l[h]) * (DROP ? a.drop.inv_keep : 1.f);
        u32x2 ow[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) ow[ct] = pack_acc<DT>(o[h][ct], inv);
        store_tile<C>(os, qrow * pitch, ow, g, stores_whole_lines(pitch, C, 0), pitch);     // rows past T are dropped
        const float pad = qrow >= tv ? kMaskValue : 0.f;
        if (g == 0)
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint((m[h] + __builtin_amdgcn_logf(l[h])) * kLn2 + pad), ls, qrow * 4, 0, 0);
    }
}

// =============================================================================
// Backward, query side: delta = rowsum(dO * O) (written to `delta`) and dQ
// =============================================================================
// A workgroup owns 4 * QT query tiles, QT to a wave, whose Q, dO and O rows go from memory straight into registers,
// and walks the keys in chunks of 4 tiles (K and V through LDS, the next chunk in flight behind the current one).
// dQ^T += K^T dS^T runs two key tiles at a time on the 32-deep product.  A padded query row's -100 is folded into
// its LSE once; chunks whose keys all count skip the masks.
template <class DT, int C, bool DROP, int QT>
__global__ void __launch_bounds__(kThreads)
global_dq_kernel(char *__restrict__ dq, float *__restrict__ delta, const char *__restrict__ q,
                 const char *__restrict__ k, const char *__restrict__ v, const char *__restrict__ out,
                 const char *__restrict__ dout, const float *__restrict__ lse, const int32_t *__restrict__ t_valid,
                 uint32_t items, GlobalArgs a) {
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    constexpr int kStep = region_bytes<C>(kStripTiles);
    fetch_args_now(dq, delta, q, k, v, out, dout, lse, t_valid, items, a.T, a.H, a.strips, a.strips_magic, a.heads_magic,
                   a.pitch, a.scale);
    if constexpr (DROP) fetch_args_now(a.drop.threshold, a.drop.seed_lo, a.drop.seed_hi, a.drop.inv_keep);
    extern __shared__ __attribute__((aligned(16))) char smem[];          // 4 * kStep bytes: K and V of two chunks
    LDS_PTR(char) kv_lds = (LDS_PTR(char))smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, n = lane & 15;
    const uint32_t item = xcd_item(blockIdx.x, items);
    const uint32_t b = div_by(item, a.strips, a.strips_magic);
    const int strip = (int)(item - b * a.strips);
    const uint32_t sample = div_by(b, a.H, a.heads_magic);
    const int T = a.T, tiles = (T + 15) >> 4;

    const int64_t seq_off = (int64_t)b * T * a.pitch;
    const Rsrc qs = make_rsrc(q + seq_off, T * a.pitch), ks = make_rsrc(k + seq_off, T * a.pitch);
    const Rsrc vs = make_rsrc(v + seq_off, T * a.pitch), os = make_rsrc(out + seq_off, T * a.pitch);
    const Rsrc gs = make_rsrc(dout + seq_off, T * a.pitch), dqs = make_rsrc(dq + seq_off, T * a.pitch);
    const Rsrc ls = make_rsrc(lse + (int64_t)b * T, T * 4), ds = make_rsrc(delta + (int64_t)b * T, T * 4);
    const int lane_off = direct_lane_offset<C>(wave, lane, a.pitch, a.pitch);
    stage_direct<C, kStripTiles, kReadShared>(ks, 0, kv_lds, kStripTiles, wave, lane_off, a.pitch);
    stage_direct<C, kStripTiles, kReadShared>(vs, 0, kv_lds + kStep, kStripTiles, wave, lane_off, a.pitch);
    int qt[QT];                                             // this wave's query tiles
    RowOperand<C> qop[QT], gop[QT], oop[QT];
    float lse_row[QT];
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        qt[h] = kStripTiles * (QT * strip + h) + wave;
        const int at = 16 * qt[h] * a.pitch;
        load_rows<C, kReadShared>(qop[h], qs, at, a.pitch, a.pitch, lane);
        load_rows<C, kReadShared>(gop[h], gs, at, a.pitch, a.pitch, lane);
        load_rows<C, kReadOnce>(oop[h], os, at, a.pitch, a.pitch, lane);
        lse_row[h] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ls, (16 * qt[h] + n) * 4, 0, 0));
    }
    int tv = T;
    if (t_valid) tv = max(0, min(T, t_valid[sample]));
    const float scale2 = a.scale * kLog2e, mask2 = kMaskValue * kLog2e;

    RowLane<C> row_lane;
    TrLane<C> tr_lane;
    row_lane.init(0, lane);
    tr_lane.init(0, lane);
    f32x4 acc[QT][CT];
    float dl[QT], ref[QT];              // ref: minus the row's LSE in the log2 domain, a padded row's -100 taken out of it
    bool row_masked[QT];
    uint32_t drop_key[QT];
    wait_direct();
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        const int qrow = 16 * qt[h] + n;
        dl[h] = xor_sum(dot_lane<DT, C>(gop[h], oop[h]));   // lane (n, g) holds a quarter of row n's channels
        row_masked[h] = qrow >= tv;
        ref[h] = (row_masked[h] ? mask2 : 0.f) - lse_row[h] * kLog2e;
        // With dropout mask D (0 or 1/(1-p)): O = (D*P) V, so dP = D * (dO . V^T) and delta = rowsum(dO * O) as before.
        drop_key[h] = DROP ? dropout_row_key((uint64_t)b * T + qrow, a.drop) : 0u;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[h][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // one chunk of keys; `whole`: all of its 64 keys exist and count
    auto chunk = [&](auto whole, int c0, LDS_PTR(char) k_lds, LDS_PTR(char) v_lds) {
        constexpr bool kWhole = decltype(whole)::value;
        const int nk = kWhole ? kStripTiles : min(kStripTiles, tiles - c0);
#pragma unroll
        for (int kt = 0; kt < kStripTiles; kt += 2) {
            if (kt >= nk) continue;
            u32x4 db[QT];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (kt + j < nk) {
                    RowOperand<C> kop, vop;
                    read_rows<C>(kop, k_lds + (kt + j) * LL::kTileBytes, row_lane);
                    read_rows<C>(vop, v_lds + (kt + j) * LL::kTileBytes, row_lane);
#pragma unroll
                    for (int h = 0; h < QT; ++h) {
                        const f32x4 s = dot_rows_mma<DT, C>(kop, qop[h]);
                        const f32x4 dp = dot_rows_mma<DT, C>(vop, gop[h]);
                        float dsv[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int key = 16 * (c0 + kt + j) + 4 * g + r;
                            float z = __builtin_fmaf(s[r], scale2, ref[h]);
                            if constexpr (!kWhole) z += (key >= tv && !row_masked[h]) ? mask2 : 0.f;
                            const float p = kWhole || key < T ? __builtin_amdgcn_exp2f(z) : 0.f;
                            float dpr = dp[r];
                            if constexpr (DROP) dpr *= dropout_keeps(drop_key[h], key, a.drop) ? a.drop.inv_keep : 0.f;
                            dsv[r] = p * (dpr - dl[h]);
                        }
                        db[h][2 * j] = Mma<DT>::pack(dsv[0], dsv[1]);
                        db[h][2 * j + 1] = Mma<DT>::pack(dsv[2], dsv[3]);
                    }
                } else {
#pragma unroll
                    for (int h = 0; h < QT; ++h) db[h][2 * j] = db[h][2 * j + 1] = 0u;     // against the zeros staged past the sequence
                }
            }
            LDS_PTR(char) blk = k_lds + kt * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const u32x2 k0 = read_tr(blk + tr_lane.off[ct]), k1 = read_tr(blk + LL::kTileBytes + tr_lane.off[ct]);
                const u32x4 kk = {k0.x, k0.y, k1.x, k1.y};
#pragma unroll
                for (int h = 0; h < QT; ++h) acc[h][ct] = Mma<DT>::k32(kk, db[h], acc[h][ct]);
            }
        }
    };
    const int whole_keys = min(T, tv);
    int at = 0;                                             // byte offset of the chunk's pair of regions: 0 or 2 * kStep
    auto step = [&](auto whole, int c0) {
        wait_direct();
        barrier_lds();      // this chunk has landed, and every wave is done with the one before, whose regions the next takes
        if (c0 + kStripTiles < tiles) {
            LDS_PTR(char) next = kv_lds + (at ^ 2 * kStep);
            stage_direct<C, kStripTiles, kReadShared>(ks, 16 * (c0 + kStripTiles), next, kStripTiles, wave, lane_off, a.pitch);
            stage_direct<C, kStripTiles, kReadShared>(vs, 16 * (c0 + kStripTiles), next + kStep, kStripTiles, wave, lane_off, a.pitch);
        }
        chunk(whole, c0, kv_lds + at, kv_lds + at + kStep);
        at ^= 2 * kStep;
    };
    int c0 = 0;
    for (; 16 * (c0 + kStripTiles) <= whole_keys; c0 += kStripTiles) step(std::true_type{}, c0);
    for (; c0 < tiles; c0 += kStripTiles) step(std::false_type{}, c0);

#pragma unroll
    for (int h = 0; h < QT; ++h) {
        if (qt[h] >= tiles) break;
        const int qrow = 16 * qt[h] + n;
        u32x2 qw[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) qw[ct] = pack_acc<DT>(acc[h][ct], a.scale);
        store_tile<C>(dqs, qrow * a.pitch, qw, g, stores_whole_lines(a.pitch, C, 0), a.pitch);
        if (g == 0) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(dl[h]), ds, qrow * 4, 0, 0);
    }
}

// =============================================================================
// Backward, key side: dK and dV
// =============================================================================
// A workgroup owns 4 * QT key tiles, QT to a wave, whose K and V rows go from memory straight into registers, and
// walks the queries in chunks of 4 tiles (Q, dO, LSE and delta through LDS, double-buffered).  The score product is
// taken with Q and K swapped, so that P and dS come out as B operands; dV^T += dO^T P and dK^T += Q^T dS run two
// query tiles at a time on the 32-deep product.
template <class DT, int C, bool DROP, int QT>
__global__ void __launch_bounds__(kThreads)
global_dkv_kernel(char *__restrict__ dk, char *__restrict__ dv, const char *__restrict__ q, const char *__restrict__ k,
                  const char *__restrict__ v, const char *__restrict__ dout, const float *__restrict__ lse,
                  const float *__restrict__ delta, const int32_t *__restrict__ t_valid, uint32_t items, GlobalArgs a) {
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    constexpr int kStep = region_bytes<C>(kStripTiles);
    constexpr int kRows = 16 * kStripTiles;                 // rows of a chunk: one lse / delta value each
    constexpr int kBuf = 2 * kStep + 2 * kRows * 4;         // Q, dO, lse, delta of one chunk
    fetch_args_now(dk, dv, q, k, v, dout, lse, delta, t_valid, items, a.T, a.H, a.strips, a.strips_magic, a.heads_magic,
                   a.pitch, a.scale);
    if constexpr (DROP) fetch_args_now(a.drop.threshold, a.drop.seed_lo, a.drop.seed_hi, a.drop.inv_keep);
    extern __shared__ __attribute__((aligned(16))) char smem[];          // 2 * kBuf bytes
    LDS_PTR(char) buf_lds = (LDS_PTR(char))smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, n = lane & 15;
    const uint32_t item = xcd_item(blockIdx.x, items);
    const uint32_t b = div_by(item, a.strips, a.strips_magic);
    const int strip = (int)(item - b * a.strips);
    const uint32_t sample = div_by(b, a.H, a.heads_magic);
    const int T = a.T, tiles = (T + 15) >> 4;

    const int64_t seq_off = (int64_t)b * T * a.pitch;
    const Rsrc qs = make_rsrc(q + seq_off, T * a.pitch), ks = make_rsrc(k + seq_off, T * a.pitch);
    const Rsrc vs = make_rsrc(v + seq_off, T * a.pitch), gs = make_rsrc(dout + seq_off, T * a.pitch);
    const Rsrc dks = make_rsrc(dk + seq_off, T * a.pitch), dvs = make_rsrc(dv + seq_off, T * a.pitch);
    const Rsrc ls = make_rsrc(lse + (int64_t)b * T, T * 4), ds = make_rsrc(delta + (int64_t)b * T, T * 4);
    const int lane_off = direct_lane_offset<C>(wave, lane, a.pitch, a.pitch);
    auto stage = [&](int c0, LDS_PTR(char) buf) {           // chunk of queries c0 .. c0 + 3 into one buffer
        stage_direct<C, kStripTiles, kReadShared>(qs, 16 * c0, buf, kStripTiles, wave, lane_off, a.pitch);
        stage_direct<C, kStripTiles, kReadShared>(gs, 16 * c0, buf + kStep, kStripTiles, wave, lane_off, a.pitch);
        if (wave == 0) load_to_lds<4, 0>(ls, buf + 2 * kStep, (16 * c0 + lane) * 4);            // rows past T: zeros
        if (wave == 1) load_to_lds<4, 0>(ds, buf + 2 * kStep + kRows * 4, (16 * c0 + lane) * 4);
    };
    stage(0, buf_lds);
    int kt_own[QT];                                         // this wave's key tiles
    RowOperand<C> kop[QT], vop[QT];
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        kt_own[h] = kStripTiles * (QT * strip + h) + wave;
        load_rows<C, kReadShared>(kop[h], ks, 16 * kt_own[h] * a.pitch, a.pitch, a.pitch, lane);
        load_rows<C, kReadShared>(vop[h], vs, 16 * kt_own[h] * a.pitch, a.pitch, a.pitch, lane);
    }
    int tv = T;
    if (t_valid) tv = max(0, min(T, t_valid[sample]));
    const float scale2 = a.scale * kLog2e, mask2 = kMaskValue * kLog2e;

    RowLane<C> row_lane;
    TrLane<C> tr_lane;
    row_lane.init(0, lane);
    tr_lane.init(0, lane);
    f32x4 acck[QT][CT], accv[QT][CT];
    bool keys_count = true;             // all keys of this wave's tiles are valid ones
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        keys_count = keys_count && 16 * kt_own[h] + 16 <= tv;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acck[h][ct] = accv[h][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // one chunk of queries; `whole`: all of its 64 rows exist and count, and so do this wave's keys
    auto chunk = [&](auto whole, int c0, LDS_PTR(char) buf) {
        constexpr bool kWhole = decltype(whole)::value;
        LDS_PTR(char) q_lds = buf;
        LDS_PTR(char) g_lds = buf + kStep;
        LDS_PTR(float) lse_lds = (LDS_PTR(float))(buf + 2 * kStep);
        LDS_PTR(float) del_lds = lse_lds + kRows;
        const int nq = kWhole ? kStripTiles : min(kStripTiles, tiles - c0);      // query tiles in this chunk
#pragma unroll
        for (int qi = 0; qi < kStripTiles; qi += 2) {
            if (qi >= nq) continue;
            u32x4 pb[QT], db[QT];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (qi + j < nq) {
                    RowOperand<C> qop, gop;
                    read_rows<C>(qop, q_lds + (qi + j) * LL::kTileBytes, row_lane);
                    read_rows<C>(gop, g_lds + (qi + j) * LL::kTileBytes, row_lane);
                    const f32x4 lse4 = *reinterpret_cast<LDS_PTR(f32x4)>(lse_lds + 16 * (qi + j) + 4 * g);
                    const f32x4 del4 = *reinterpret_cast<LDS_PTR(f32x4)>(del_lds + 16 * (qi + j) + 4 * g);
#pragma unroll
                    for (int h = 0; h < QT; ++h) {
                        const int key = 16 * kt_own[h] + n;
                        const f32x4 s = dot_rows_mma<DT, C>(qop, kop[h]);        // [query 4g+r][key n]
                        const f32x4 dp = dot_rows_mma<DT, C>(gop, vop[h]);
                        float p[4], dsv[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int qrow = 16 * (c0 + qi + j) + 4 * g + r;
                            float z = __builtin_fmaf(s[r], scale2, -kLog2e * lse4[r]);
                            if constexpr (!kWhole) z += (key >= tv || qrow >= tv) ? mask2 : 0.f;
                            p[r] = kWhole || qrow < T ? __builtin_amdgcn_exp2f(z) : 0.f;     // rows past the sequence do not exist
                            float f = 1.f;     // dropout: dP is masked, and dV takes the probability as the forward used it
                            if constexpr (DROP)
                                f = dropout_keeps(dropout_row_key((uint64_t)b * T + qrow, a.drop), key, a.drop) ? a.drop.inv_keep : 0.f;
                            dsv[r] = p[r] * (dp[r] * f - del4[r]);
                            p[r] *= f;
                        }
                        pb[h][2 * j] = Mma<DT>::pack(p[0], p[1]);
                        pb[h][2 * j + 1] = Mma<DT>::pack(p[2], p[3]);
                        db[h][2 * j] = Mma<DT>::pack(dsv[0], dsv[1]);
                        db[h][2 * j + 1] = Mma<DT>::pack(dsv[2], dsv[3]);
                    }
                } else {
#pragma unroll
                    for (int h = 0; h < QT; ++h) pb[h][2 * j] = pb[h][2 * j + 1] = db[h][2 * j] = db[h][2 * j + 1] = 0u;
                }
            }
            LDS_PTR(char) qtile = q_lds + qi * LL::kTileBytes;
            LDS_PTR(char) gtile = g_lds + qi * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const u32x2 g0 = read_tr(gtile + tr_lane.off[ct]), g1 = read_tr(gtile + LL::kTileBytes + tr_lane.off[ct]);
                const u32x2 q0 = read_tr(qtile + tr_lane.off[ct]), q1 = read_tr(qtile + LL::kTileBytes + tr_lane.off[ct]);
                const u32x4 gg = {g0.x, g0.y, g1.x, g1.y}, qq = {q0.x, q0.y, q1.x, q1.y};
#pragma unroll
                for (int h = 0; h < QT; ++h) {
                    accv[h][ct] = Mma<DT>::k32(gg, pb[h], accv[h][ct]);
                    acck[h][ct] = Mma<DT>::k32(qq, db[h], acck[h][ct]);
                }
            }
        }
    };
    const int whole_rows = keys_count ? min(T, tv) : 0;
    int at = 0;
    auto step = [&](auto whole, int c0) {
        wait_direct();
        barrier_lds();      // this chunk has landed, and every wave is done with the one before, whose buffer the next takes
        if (c0 + kStripTiles < tiles) stage(c0 + kStripTiles, buf_lds + (at ^ kBuf));
        chunk(whole, c0, buf_lds + at);
        at ^= kBuf;
    };
    int c0 = 0;
    for (; 16 * (c0 + kStripTiles) <= whole_rows; c0 += kStripTiles) step(std::true_type{}, c0);
    for (; c0 < tiles; c0 += kStripTiles) step(std::false_type{}, c0);

    const bool stream = stores_whole_lines(a.pitch, C, 0);
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        if (kt_own[h] >= tiles) break;
        const int key = 16 * kt_own[h] + n;
        u32x2 kw[CT], vw[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            kw[ct] = pack_acc<DT>(acck[h][ct], a.scale);
            vw[ct] = pack_acc<DT>(accv[h][ct], 1.f);
        }
        store_tile<C>(dks, key * a.pitch, kw, g, stream, a.pitch);      // rows past T are dropped
        store_tile<C>(dvs, key * a.pitch, vw, g, stream, a.pitch);
    }
}

// =============================================================================
// Backward for sequences of up to 128 rows: one workgroup per sequence and ONE kernel.  Q, K, V and dO sit whole in
// LDS behind a single barrier.  Every wave first takes query tiles (delta and dQ, as global_dq_kernel), leaves delta
// in LDS for the others, and then, behind a second barrier, key tiles (dK and dV, as global_dkv_kernel).  Each input
// is read from memory once and delta never leaves the chip.
// =============================================================================
template <class DT, int C, bool DROP, int TILES, int QT>
__global__ void __launch_bounds__(64 * TILES / QT)
global_bwd_short_kernel(char *__restrict__ dq, char *__restrict__ dk, char *__restrict__ dv, const char *__restrict__ q,
                        const char *__restrict__ k, const char *__restrict__ v, const char *__restrict__ out,
                        const char *__restrict__ dout, const float *__restrict__ lse, const int32_t *__restrict__ t_valid,
                        GlobalArgs a) {
    using LL = Lds<C>;
    constexpr int CT = C / 16, kW = TILES / QT;       // waves of the workgroup, QT query / key tiles each
    constexpr int kRows = 16 * TILES;
    fetch_args_now(dq, dk, dv, q, k, v, out, dout, lse, t_valid, a.T, a.H, a.heads_magic, a.pitch, a.scale);
    if constexpr (DROP) fetch_args_now(a.drop.threshold, a.drop.seed_lo, a.drop.seed_hi, a.drop.inv_keep);
    const int T = a.T, tiles = (T + 15) >> 4, pitch = a.pitch;
    const int region = region_bytes<C>(tiles);
    extern __shared__ __attribute__((aligned(16))) char smem[];          // 4 * region + 2 * kRows * 4 bytes
    LDS_PTR(char) q_lds = (LDS_PTR(char))smem;
    LDS_PTR(char) g_lds = q_lds + region;                   // dO
    LDS_PTR(char) k_lds = g_lds + region;
    LDS_PTR(char) v_lds = k_lds + region;
    LDS_PTR(float) lse_lds = (LDS_PTR(float))(v_lds + region);
    LDS_PTR(float) del_lds = lse_lds + kRows;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, n = lane & 15;
    const uint32_t b = blockIdx.x;
    const int64_t seq_off = (int64_t)((uint64_t)b * (uint32_t)(T * pitch));
    const Rsrc qs = make_rsrc(q + seq_off, T * pitch), gs = make_rsrc(dout + seq_off, T * pitch);
    const Rsrc ks = make_rsrc(k + seq_off, T * pitch), vs = make_rsrc(v + seq_off, T * pitch);
    const Rsrc os = make_rsrc(out + seq_off, T * pitch), ls = make_rsrc(lse + (int64_t)b * T, T * 4);
    const int lane_off = direct_lane_offset<C>(wave, lane, pitch, pitch);
    stage_direct<C, TILES, kReadOnce, kW>(qs, 0, q_lds, tiles, wave, lane_off, pitch);
    stage_direct<C, TILES, kReadOnce, kW>(gs, 0, g_lds, tiles, wave, lane_off, pitch);
    stage_direct<C, TILES, kReadOnce, kW>(ks, 0, k_lds, tiles, wave, lane_off, pitch);
    stage_direct<C, TILES, kReadOnce, kW>(vs, 0, v_lds, tiles, wave, lane_off, pitch);
    if (wave < kRows / 64) load_to_lds<4, 0>(ls, (LDS_PTR(char))(lse_lds + 64 * wave), (64 * wave + lane) * 4);     // rows past T: zeros
    // this wave's own tiles (as queries first, as keys later); one past the sequence's last computes on that one and stores nothing
    int own[QT];
    RowOperand<C> oop[QT];
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        own[h] = min(wave + kW * h, tiles - 1);
        load_rows<C, kReadOnce>(oop[h], os, 16 * own[h] * pitch, pitch, pitch, lane);
    }
    __builtin_amdgcn_sched_barrier(0);

    const uint32_t sample = div_by(b, a.H, a.heads_magic);
    int tv = T;
    if (t_valid) tv = max(0, min(T, t_valid[sample]));
    const float scale2 = a.scale * kLog2e, mask2 = kMaskValue * kLog2e;
    RowLane<C> row_lane;
    TrLane<C> tr_lane;
    row_lane.init(0, lane);
    tr_lane.init(0, lane);
    wait_direct();
    barrier_lds();

    // ---- queries: delta and dQ -------------------------------------------------------------------------------
    {
        RowOperand<C> qop[QT], gop[QT];
        float dl[QT], lse2[QT];
        uint32_t drop_key[QT];
        f32x4 acc[QT][CT];
#pragma unroll
        for (int h = 0; h < QT; ++h) {
            const int qrow = 16 * own[h] + n;
            read_rows<C>(qop[h], q_lds + own[h] * LL::kTileBytes, row_lane);
            read_rows<C>(gop[h], g_lds + own[h] * LL::kTileBytes, row_lane);
            dl[h] = xor_sum(dot_lane<DT, C>(gop[h], oop[h]));       // lane (n, g) holds a quarter of row n's channels
            lse2[h] = lse_lds[qrow] * kLog2e;
            if (g == 0) del_lds[qrow] = dl[h];
            // With dropout mask D (0 or 1/(1-p)): O = (D*P) V, so dP = D * (dO . V^T) and delta = rowsum(dO * O) as before.
            drop_key[h] = DROP ? dropout_row_key((uint64_t)b * T + qrow, a.drop) : 0u;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) acc[h][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int kt = 0; kt < TILES; ++kt) {
            if (kt >= tiles) continue;
            RowOperand<C> kop, vop;
            read_rows<C>(kop, k_lds + kt * LL::kTileBytes, row_lane);
            read_rows<C>(vop, v_lds + kt * LL::kTileBytes, row_lane);
            u32x2 db[QT];
#pragma unroll
            for (int h = 0; h < QT; ++h) {
                const bool row_masked = 16 * own[h] + n >= tv;
                const f32x4 sc = dot_rows_mma<DT, C>(kop, qop[h]);
                const f32x4 dp = dot_rows_mma<DT, C>(vop, gop[h]);
                float dsv[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = 16 * kt + 4 * g + r;
                    const float z = sc[r] * scale2 - lse2[h] + ((key >= tv || row_masked) ? mask2 : 0.f);
                    const float p = key < T ? __builtin_amdgcn_exp2f(z) : 0.f;
                    float dpr = dp[r];
                    if constexpr (DROP) dpr *= dropout_keeps(drop_key[h], key, a.drop) ? a.drop.inv_keep : 0.f;
                    dsv[r] = p * (dpr - dl[h]);
                }
                db[h] = u32x2{Mma<DT>::pack(dsv[0], dsv[1]), Mma<DT>::pack(dsv[2], dsv[3])};
            }
            LDS_PTR(char) blk = k_lds + kt * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const auto kt_t = read_tr(blk + tr_lane.off[ct]);
#pragma unroll
                for (int h = 0; h < QT; ++h) acc[h][ct] = Mma<DT>::k16(kt_t, db[h], acc[h][ct]);
            }
        }
        const Rsrc dqs = make_rsrc(dq + seq_off, T * pitch);
#pragma unroll
        for (int h = 0; h < QT; ++h) {
            if (wave + kW * h >= tiles) break;
            u32x2 qw[CT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) qw[ct] = pack_acc<DT>(acc[h][ct], a.scale);
            store_tile<C>(dqs, (16 * own[h] + n) * pitch, qw, g, stores_whole_lines(pitch, C, 0), pitch);   // rows past T are dropped
        }
    }
    barrier_lds();                                          // every row's delta is in LDS

    // ---- keys: dK and dV -------------------------------------------------------------------------------------
    RowOperand<C> kop[QT], vop[QT];
    f32x4 acck[QT][CT], accv[QT][CT];
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        read_rows<C>(kop[h], k_lds + own[h] * LL::kTileBytes, row_lane);
        read_rows<C>(vop[h], v_lds + own[h] * LL::kTileBytes, row_lane);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acck[h][ct] = accv[h][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int qi = 0; qi < TILES; ++qi) {
        if (qi >= tiles) continue;
        RowOperand<C> qop, gop;
        read_rows<C>(qop, q_lds + qi * LL::kTileBytes, row_lane);
        read_rows<C>(gop, g_lds + qi * LL::kTileBytes, row_lane);
        const f32x4 lse4 = *reinterpret_cast<LDS_PTR(f32x4)>(lse_lds + 16 * qi + 4 * g);
        const f32x4 del4 = *reinterpret_cast<LDS_PTR(f32x4)>(del_lds + 16 * qi + 4 * g);
        u32x2 pb[QT], db[QT];
#pragma unroll
        for (int h = 0; h < QT; ++h) {
            const int key = 16 * own[h] + n;
            const bool col_masked = key >= tv;
            const f32x4 sc = dot_rows_mma<DT, C>(qop, kop[h]);       // [query 4g+r][key n]
            const f32x4 dp = dot_rows_mma<DT, C>(gop, vop[h]);
            float p[4], dsv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int qrow = 16 * qi + 4 * g + r;
                const float z = sc[r] * scale2 - lse4[r] * kLog2e + ((col_masked || qrow >= tv) ? mask2 : 0.f);
                p[r] = qrow < T ? __builtin_amdgcn_exp2f(z) : 0.f;   // rows past the sequence do not exist
                float f = 1.f;             // dropout: dP is masked, and dV takes the probability as the forward used it
                if constexpr (DROP)
                    f = dropout_keeps(dropout_row_key((uint64_t)b * T + qrow, a.drop), key, a.drop) ? a.drop.inv_keep : 0.f;
                dsv[r] = p[r] * (dp[r] * f - del4[r]);
                p[r] *= f;
            }
            pb[h] = u32x2{Mma<DT>::pack(p[0], p[1]), Mma<DT>::pack(p[2], p[3])};
            db[h] = u32x2{Mma<DT>::pack(dsv[0], dsv[1]), Mma<DT>::pack(dsv[2], dsv[3])};
        }
        LDS_PTR(char) qtile = q_lds + qi * LL::kTileBytes;
        LDS_PTR(char) gtile = g_lds + qi * LL::kTileBytes;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const auto g_t = read_tr(gtile + tr_lane.off[ct]), q_t = read_tr(qtile + tr_lane.off[ct]);
#pragma unroll
            for (int h = 0; h < QT; ++h) {
                accv[h][ct] = Mma<DT>::k16(g_t, pb[h], accv[h][ct]);
                acck[h][ct] = Mma<DT>::k16(q_t, db[h], acck[h][ct]);
            }
        }
    }
    const Rsrc dks = make_rsrc(dk + seq_off, T * pitch), dvs = make_rsrc(dv + seq_off, T * pitch);
    const bool stream = stores_whole_lines(pitch, C, 0);
#pragma unroll
    for (int h = 0; h < QT; ++h) {
        if (wave + kW * h >= tiles) break;
        u32x2 kw[CT], vw[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            kw[ct] = pack_acc<DT>(acck[h][ct], a.scale);
            vw[ct] = pack_acc<DT>(accv[h][ct], 1.f);
        }
        store_tile<C>(dks, (16 * own[h] + n) * pitch, kw, g, stream, pitch);      // rows past T are dropped
        store_tile<C>(dvs, (16 * own[h] + n) * pitch, vw, g, stream, pitch);
    }
}

// ----------------------------------------------------------------------------- launchers
inline bool global_ok(const Geom &g, GlobalArgs &a, int64_t &items) {
    if (g.C > 128 || g.T > (1 << 28) / g.C) return false;
    const int tiles = (int)((g.T + 15) / 16);
    a.T = (int)g.T;
    a.H = g.H;
    a.strips = (tiles + kStripTiles - 1) / kStripTiles;
    items = g.B * a.strips;
    if (items > 0x7fffff00LL || !div_magic_ok(items, a.strips) || !div_magic_ok(g.B, g.H)) return false;
    a.strips_magic = div_magic(a.strips);
    a.heads_magic = div_magic(g.H);
    a.pitch = 2 * g.C;
    a.drop = g.drop;
    return true;
}

template <class DT, int C>
int launch_global_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const int32_t *t_valid,
                      const Geom &g, float scale, hipStream_t s) {
    GlobalArgs a;
    int64_t items;
    if (!global_ok(g, a, items)) return NA1D_ERR_UNSUPPORTED;
    a.scale = scale;
    const char *dt_name = DT::tag == NA1D_BF16 ? "BF16" : "FP16", *drop_name = g.drop.threshold ? "true" : "false";
    if (g.T <= 16 * kShortTiles) {
        // sequences of up to 4 tiles: a tile to each of the 4 waves; longer ones: two, which read every key and value
        // operand half as often
        const bool small = g.T <= 64;
        const size_t lds = 2 * (size_t)region_bytes<C>((int)(g.T + 15) / 16);
        auto go = [&](auto kern) {
            if (!allow_lds(kern, lds)) return (int)NA1D_ERR_LAUNCH;
            note_kernel_as("global_fwd_short_kernel<%s, %d, %s, %s>", dt_name, C, drop_name, small ? "4, 1" : "8, 2");
            launch_kernel(kern, (unsigned)g.B, lds, s, (char *)out, lse, (const char *)q, (const char *)k, (const char *)v,
                          t_valid, a);
            return launch_status();
        };
        if (g.drop.threshold)
            return small ? go(global_fwd_short_kernel<DT, C, true, 4, 1>) : go(global_fwd_short_kernel<DT, C, true, 8, 2>);
        return small ? go(global_fwd_short_kernel<DT, C, false, 4, 1>) : go(global_fwd_short_kernel<DT, C, false, 8, 2>);
    }
    // two query tiles to a wave where that still leaves every CU several workgroups and at most one workgroup in seven
    // or more half empty
    const int64_t strips2 = (a.strips + 1) / 2;
    const bool two = (a.strips % 2 == 0 || a.strips >= 7) && g.B * strips2 >= 4 * 256 && div_magic_ok(g.B * strips2, strips2);
    if (two) {
        a.strips = (int)strips2;
        a.strips_magic = div_magic(a.strips);
        items = g.B * strips2;
    }
    const size_t lds = 4 * (size_t)region_bytes<C>(kStripTiles);
    auto go = [&](auto kern) {
        if (!allow_lds(kern, lds)) return (int)NA1D_ERR_LAUNCH;
        note_kernel_as("global_fwd_kernel<%s, %d, %s, %d>", dt_name, C, drop_name, two ? 2 : 1);
        launch_kernel(kern, (unsigned)items, lds, s, (char *)out, lse, (const char *)q, (const char *)k, (const char *)v, t_valid,
                      (uint32_t)items, a);
        return launch_status();
    };
    if (g.drop.threshold) return two ? go(global_fwd_kernel<DT, C, true, 2>) : go(global_fwd_kernel<DT, C, true, 1>);
    return two ? go(global_fwd_kernel<DT, C, false, 2>) : go(global_fwd_kernel<DT, C, false, 1>);
}

template <class DT, int C>
int launch_global_bwd(void *dq, void *dk, void *dv, float *delta, const void *q, const void *k, const void *v,
                      const void *out, const void *dout, const float *lse, const int32_t *t_valid, const Geom &g,
                      float scale, hipStream_t s) {
    GlobalArgs a;
    int64_t items;
    if (!global_ok(g, a, items)) return NA1D_ERR_UNSUPPORTED;
    a.scale = scale;
    if (g.T <= 16 * kShortTiles) {
        const int tiles_max = g.T <= 64 ? 4 : 8;            // a wave per tile either way
        const size_t lds = 4 * (size_t)region_bytes<C>((int)(g.T + 15) / 16) + 2 * 16 * tiles_max * sizeof(float);
        auto go = [&](auto kern) {
            if (!allow_lds(kern, lds)) return (int)NA1D_ERR_LAUNCH;
            note_kernel_as("global_bwd_short_kernel<%s, %d, %s, %d, 1>", DT::tag == NA1D_BF16 ? "BF16" : "FP16", C,
                           g.drop.threshold ? "true" : "false", tiles_max);
            launch_kernel_block(kern, (unsigned)g.B, 64u * tiles_max, lds, s, (char *)dq, (char *)dk, (char *)dv, (const char *)q,
                                (const char *)k, (const char *)v, (const char *)out, (const char *)dout, lse, t_valid, a);
            return launch_status();
        };
        if (g.drop.threshold)
            return tiles_max == 4 ? go(global_bwd_short_kernel<DT, C, true, 4, 1>) : go(global_bwd_short_kernel<DT, C, true, 8, 1>);
        return tiles_max == 4 ? go(global_bwd_short_kernel<DT, C, false, 4, 1>) : go(global_bwd_short_kernel<DT, C, false, 8, 1>);
    }
    // two tiles to a wave where that leaves every CU several workgroups and at most one workgroup in seven or more half empty
    const int64_t strips2 = (a.strips + 1) / 2;
    const bool two = (a.strips % 2 == 0 || a.strips >= 7) && g.B * strips2 >= 4 * 256 && div_magic_ok(g.B * strips2, strips2);
    if (two) {
        a.strips = (int)strips2;
        a.strips_magic = div_magic(a.strips);
        items = g.B * strips2;
    }
    constexpr size_t dq_lds = 4 * (size_t)region_bytes<C>(kStripTiles);
    constexpr size_t dkv_lds = 2 * (2 * (size_t)region_bytes<C>(kStripTiles) + 2 * 16 * kStripTiles * sizeof(float));
    auto go = [&](auto dq_kern, auto dkv_kern) {
        if (!allow_lds(dq_kern, dq_lds) || !allow_lds(dkv_kern, dkv_lds)) return (int)NA1D_ERR_LAUNCH;
        // the pair of profiling events, if set, spans both kernels
        note_kernel_as("global_dq_kernel + global_dkv_kernel<%s, %d, %s, %d>", DT::tag == NA1D_BF16 ? "BF16" : "FP16", C,
                       g.drop.threshold ? "true" : "false", two ? 2 : 1);
        launch_kernel_span(1, dq_kern, (unsigned)items, (unsigned)kThreads, dq_lds, s, (char *)dq, delta, (const char *)q,
                           (const char *)k, (const char *)v, (const char *)out, (const char *)dout, lse, t_valid, (uint32_t)items, a);
        launch_kernel_span(2, dkv_kern, (unsigned)items, (unsigned)kThreads, dkv_lds, s, (char *)dk, (char *)dv,
                           (const char *)q, (const char *)k, (const char *)v, (const char *)dout, lse, delta, t_valid,
                           (uint32_t)items, a);
        return launch_status();
    };
    if (g.drop.threshold)
        return two ? go(global_dq_kernel<DT, C, true, 2>, global_dkv_kernel<DT, C, true, 2>)
                   : go(global_dq_kernel<DT, C, true, 1>, global_dkv_kernel<DT, C, true, 1>);
    return two ? go(global_dq_kernel<DT, C, false, 2>, global_dkv_kernel<DT, C, false, 2>)
               : go(global_dq_kernel<DT, C, false, 1>, global_dkv_kernel<DT, C, false, 1>);
}

int global_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const int32_t *t_valid,
               const Geom &g, float scale, int dtype, hipStream_t s) {
    NA1D_MFMA_DISPATCH(launch_global_fwd, out, lse, q, k, v, t_valid, g, scale, s);
}

int global_bwd(void *dq, void *dk, void *dv, float *delta, const void *q, const void *k, const void *v, const void *out,
               const void *dout, const float *lse, const int32_t *t_valid, const Geom &g, float scale, int dtype,
               hipStream_t s) {
    NA1D_MFMA_DISPATCH(launch_global_bwd, dq, dk, dv, delta, q, k, v, out, dout, lse, t_valid, g, scale, s);
}

}  // namespace mfma
}  // namespace na1d
