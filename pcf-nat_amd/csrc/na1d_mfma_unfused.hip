// The three un-fused NA1D primitives on the matrix cores (gfx950): band QK^T (P1),
// band . V (P2) and the inverse-neighbourhood gather (P3), with the fp32 [B,T,W]
// score tensor in memory as the reference's two-call API has it.  Tiling, LDS layout
// and operand conventions are those of na1d_mfma_core.h; the score rows of a strip are
// contiguous in memory (16*W floats per tile), so they move between HBM and LDS as
// plain 16-byte copies and are picked apart / assembled per lane inside LDS.
//
// P2 and P3 round the scores to the 16-bit dtype before the contraction, as the
// reference kernels do (bf16_ana1d_kernel.cu:305,414); accumulation is fp32.
//
// A query tile meets NBV = 2 .. 6 virtual key blocks (W up to 80); the first one starts `shift` rows before
// the tile, shift in [L, 16*NBV - 16 - R], on a 128-byte line where that is possible.
#include "na1d_mfma_core.h"

namespace na1d {
namespace mfma {

struct BandCover {
    int nbv, shift, max_tiles;   // 0 blocks: shape not covered
};
inline BandCover band_cover(const Geom &g) {
    BandCover c{0, 0, 0};
    if (g.C > 128) return c;             // head_dim is run at the next of 16, 32, 64, 128, zero-padded
    if (g.T > (1 << 29) / g.C || g.T > (1 << 29) / (4 * g.W) || g.W > NA1D_MAX_WINDOW) return c;
    c.nbv = std::max(2, (15 + g.W + 15) / 16);
    const int R = g.W - 1 - g.L, rows = std::max(1, 128 / (2 * g.C));
    const int hi = 16 * c.nbv - 16 - R, s16 = (g.L + 15) / 16 * 16, s = (g.L + rows - 1) / rows * rows;
    c.shift = s16 <= hi ? s16 : s <= hi ? s : g.L;      // whole tiles, else whole lines, else the first key
    c.max_tiles = c.nbv <= 3 ? (g.C <= 32 ? 8 : g.C <= 64 ? 4 : 2) : (g.C <= 64 ? 4 : 2);
    return c;
}
constexpr int kBandMaxTiles = 8;          // compile-time ceiling of max_tiles

// Copy `floats` fp32 values starting `first` floats into a sequence's score rows straight into LDS, one
// 1 KB chunk per wave and round (see stage_direct); the buffer resource zero-fills what lies outside the
// rows the strip needs.  `first` is a tile start, so 16-byte units never straddle the sequence's start.
// The region is padded to whole chunks (score_bytes).
inline __host__ __device__ int score_bytes(int tiles, int W) { return (tiles * 16 * W * 4 + kChunk - 1) / kChunk * kChunk; }
template <int NBV, int AUX>
__device__ inline void stage_scores(Rsrc src, int first, LDS_PTR(float) region, int tiles, int W, int wave, int lane) {
    // at most kBandMaxTiles + NBV tiles of 16 rows of W <= 16*NBV - 15 floats
    constexpr int kRounds = (((kBandMaxTiles + NBV) * 16 * (16 * NBV - 15) * 4 + kChunk - 1) / kChunk + kWaves - 1) / kWaves;
    const int chunks = score_bytes(tiles, W) / kChunk;
#pragma unroll
    for (int j = 0; j < kRounds; ++j) {
        const int c = j * kWaves + wave;
        if (c < chunks)
            load_to_lds<16, AUX>(src, (LDS_PTR(char))(region + c * (kChunk / 4)), first * 4 + c * kChunk + lane * 16);
    }
}

__device__ inline float score_at(LDS_PTR(float) rows, int row, int j, int W) {   // 0 outside the band
    const float val = rows[row * W + min(max(j, 0), W - 1)];
    return (j >= 0 && j < W) ? val : 0.f;
}

// Narrow heads and few key blocks: the key rows of a wave's two tiles (NBV + 1 tiles of them) fit its registers as well,
// and the kernel needs no staged input, no barrier and no wait but each wave's own.
template <int C, int NBV> constexpr bool qk_keys_direct() { return (NBV + 1) * (C / 8) <= 16; }
// Whether the K region of kt tiles ends with at least 64 words that its copies fill but no tile uses.
template <int C> __host__ __device__ constexpr bool qk_spare_words(int kt) { return region_bytes<C>(kt) - kt * Lds<C>::kTileBytes >= 256; }

// =============================================================================
// P1: attn[b,t,j] = sum_c a[b,t,c] * b~[b,t-L+j,c]
// =============================================================================
template <class DT, int C, int NBV>
__global__ void __launch_bounds__(kThreads)
qk_kernel(float *__restrict__ attn, const char *__restrict__ qa, const char *__restrict__ kb, uint32_t items, int T,
          int W, int L, int tiles, int nt, int strips, uint32_t strips_magic, int shift, int pitch) {
    using LL = Lds<C>;
    constexpr int MT = kBandMaxTiles;
    fetch_args_now(attn, qa, kb, items, T, W, L, tiles, nt, strips, strips_magic, shift, pitch);
    // dynamic LDS: K region of kt tiles starting sb tiles before the strip, two 16 x W fp32 tiles per wave (and 64 words for the results that belong to no slot, unless the K region's padding has them)
    const int sb = (shift + 15) >> 4, kt = nt - 1 + NBV + ((shift & 15) ? 1 : 0);
    extern __shared__ __attribute__((aligned(16))) char smem[];
    LDS_PTR(char) k_lds = (LDS_PTR(char))smem;
    constexpr bool kDirect = qk_keys_direct<C, NBV>();
    LDS_PTR(float) out_lds = (LDS_PTR(float))(k_lds + (kDirect ? 0 : region_bytes<C>(kt)));

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t item = xcd_item(blockIdx.x, items);
    const uint32_t b = div_by(item, strips, strips_magic);
    const int strip = (int)(item - b * strips);
    const int i0 = strip * nt, i1 = min(i0 + nt, tiles);
    const int g = lane >> 4, n = lane & 15;

    const int64_t seq_off = (int64_t)b * T * pitch;      // packed rows of head_dim = pitch / 2 channels
    // A wave computes two neighbouring tiles (a strip has at most eight): their query rows, which no other wave needs,
    // come straight into the registers of the matrix operand - the key rows, which three tiles share, go through LDS.
    // Not staging the query rows is worth two more workgroups on a CU at 32 channels.
    const int i = i0 + 2 * wave;
    RowOperand<C> qt[2], kr[kDirect ? NBV + 1 : 1];
    {
        const int key_bytes = min(T, 16 * (i0 - sb + kt)) * pitch, qry_bytes = min(T, 16 * i1) * pitch;
        const int lane_off = direct_lane_offset<C>(wave, lane, pitch, pitch);
        const Rsrc qs = make_rsrc(qa + seq_off, qry_bytes);
        if constexpr (kDirect) {
            const Rsrc ks = make_rsrc(kb + seq_off, T * pitch);
            // neighbouring waves ask for the same key rows at about the same time: the default policy, whatever the strips
#pragma unroll
            for (int j = 0; j <= NBV; ++j) load_rows<C, kReadShared>(kr[j], ks, (16 * (i + j) - shift) * pitch, pitch, pitch, lane);
#pragma unroll
            for (int h = 0; h < 2; ++h) load_rows<C, kReadOnce>(qt[h], qs, 16 * (i + h) * pitch, pitch, pitch, lane);
        } else if (strips == 1) {      // nobody else reads these rows
            stage_direct<C, MT + NBV, kReadOnce>(make_rsrc(kb + seq_off, key_bytes), 16 * (i0 - sb), k_lds, kt, wave, lane_off, pitch);
#pragma unroll
            for (int h = 0; h < 2; ++h) load_rows<C, kReadOnce>(qt[h], qs, 16 * (i + h) * pitch, pitch, pitch, lane);
        } else {
            stage_direct<C, MT + NBV, kReadShared>(make_rsrc(kb + seq_off, key_bytes), 16 * (i0 - sb), k_lds, kt, wave, lane_off, pitch);
#pragma unroll
            for (int h = 0; h < 2; ++h) load_rows<C, kReadShared>(qt[h], qs, 16 * (i + h) * pitch, pitch, pitch, lane);
        }
    }
    const Rsrc as = make_rsrc(attn + (int64_t)b * T * W, T * W * 4);
    RowLane<C> k_lane;
    k_lane.init(16 * sb - shift, lane);
    LDS_PTR(float) mine = out_lds + wave * 32 * W;
    // Where this lane's four results of virtual block vb go inside a 16 x W tile: slot j = 16*vb + 4g + r - shift - n + L
    // of row n, the same for every tile.  Slots outside the window are sent to a word per lane that nobody reads (one
    // set of 64 words for all waves: in the padding of the K region where the copies leave that much, else behind the
    // waves' tiles), so that every write is unconditional: twelve masked writes a tile, each behind its own branch,
    // were most of the instructions of a tile.
    const int nowhere = (int)(!kDirect && qk_spare_words<C>(kt) ? (LDS_PTR(char))k_lds + kt * LL::kTileBytes - (LDS_PTR(char))mine
                                                     : (LDS_PTR(char))(out_lds + kWaves * 32 * W) - (LDS_PTR(char))mine) + lane * 4;
    int slot_at[2][NBV][4];             // byte offsets from `mine`, for the first and the second tile of a pair
#pragma unroll
    for (int vb = 0; vb < NBV; ++vb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int j = 16 * vb + 4 * g + r - shift - n + L;
            const bool in_window = j >= 0 && j < W;
            slot_at[0][vb][r] = in_window ? (n * W + j) * 4 : nowhere;
            slot_at[1][vb][r] = in_window ? (16 * W + n * W + j) * 4 : nowhere;
            settle(slot_at[0][vb][r]);
            settle(slot_at[1][vb][r]);
        }
    if constexpr (!kDirect) {
        wait_direct();
        barrier_lds();
    }

    // A wave takes two neighbouring tiles at a time: their 32*W floats are a run of W whole 128-byte lines (where the
    // sequence's rows start on a line), which leaves as one streaming write instead of two pieces per tile that L2
    // has to merge.  The runs are written with the streaming policy also where a sequence's rows do not start on a
    // line (T*W*4 not a multiple of 128: the run then shares its first and last line with the neighbouring runs) and
    // for the single last tile: measured with 100 rows of 27 slots, where no sequence but the first is aligned, it
    // is still the faster policy (15.4 against 16.1 us), the two shared lines being a small part of a run's 27.
    static_assert(kBandMaxTiles <= 2 * kWaves, "a wave's two tiles cover the strip");
    if (i < i1) {
        const int pair = min(2, i1 - i);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (h >= pair) break;
            const int tile_bytes = (i + h - i0) * LL::kTileBytes;
#pragma unroll
            for (int vb = 0; vb < NBV; ++vb) {
                RowOperand<C> kop;
                if constexpr (kDirect)
                    kop = kr[h + vb];
                else
                    read_rows<C>(kop, k_lds + tile_bytes + vb * LL::kTileBytes, k_lane);
                const f32x4 s = dot_rows_mma<DT, C>(kop, qt[h]);
#pragma unroll
                for (int r = 0; r < 4; ++r)        // every (row, slot) is written by exactly one lane
                    *reinterpret_cast<LDS_PTR(float)>((LDS_PTR(char))mine + slot_at[h][vb][r]) = s[r];
            }
        }
        // LDS serves one wave's accesses in program order, so the other lanes' values are there when the
        // reads below execute; the fence only keeps the compiler from moving them across
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const int first = 16 * i * W;                             // floats into the sequence's score rows
        for (int u = lane; u * 4 < pair * 16 * W; u += 64)
            __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<LDS_PTR(u32x4)>(mine + u * 4), as, (first + u * 4) * 4, 0, kStoreAux);
    }
}

// =============================================================================
// P2: out[b,t,c] = sum_j attn[b,t,j] * v~[b,t-L+j,c]
// =============================================================================
template <class DT, int C, int NBV>
__global__ void __launch_bounds__(kThreads)
av_kernel(char *__restrict__ out, const float *__restrict__ attn, const char *__restrict__ v, uint32_t items, int T,
          int W, int L, int tiles, int nt, int strips, uint32_t strips_magic, int shift, int pitch) {
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    constexpr int MT = kBandMaxTiles;
    fetch_args_now(out, attn, v, items, T, W, L, tiles, nt, strips, strips_magic, shift, pitch);
    // dynamic LDS: V region of kt tiles starting sb tiles before the strip, score rows of the strip (nt*16 x W fp32)
    const int sb = (shift + 15) >> 4, kt = nt - 1 + NBV + ((shift & 15) ? 1 : 0);
    extern __shared__ __attribute__((aligned(16))) char smem[];
    LDS_PTR(char) v_lds = (LDS_PTR(char))smem;
    LDS_PTR(float) s_lds = (LDS_PTR(float))(v_lds + region_bytes<C>(kt));

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t item = xcd_item(blockIdx.x, items);
    const uint32_t b = div_by(item, strips, strips_magic);
    const int strip = (int)(item - b * strips);
    const int i0 = strip * nt, i1 = min(i0 + nt, tiles);
    const int g = lane >> 4, n = lane & 15;

    const int64_t seq_off = (int64_t)b * T * pitch;      // packed rows of head_dim = pitch / 2 channels
    {
        const int key_bytes = min(T, 16 * (i0 - sb + kt)) * pitch;
        const int lane_off = direct_lane_offset<C>(wave, lane, pitch, pitch);
        if (strips == 1)        // nobody else reads these rows
            stage_direct<C, MT + NBV, kReadOnce>(make_rsrc(v + seq_off, key_bytes), 16 * (i0 - sb), v_lds, kt, wave, lane_off, pitch);
        else
            stage_direct<C, MT + NBV, kReadShared>(make_rsrc(v + seq_off, key_bytes), 16 * (i0 - sb), v_lds, kt, wave, lane_off, pitch);
        // the strip's own score rows: read once (at most the line at either end is shared with a neighbour)
        stage_scores<NBV, kReadOnce>(make_rsrc(attn + (int64_t)b * T * W, min(T, 16 * i1) * W * 4), 16 * i0 * W, s_lds, nt, W, wave, lane);
    }
    const Rsrc os = make_rsrc(out + seq_off, T * pitch);
    TrLane<C> v_lane;
    v_lane.init(16 * sb - shift, lane);
    wait_direct();
    __syncthreads();

    for (int i = i0 + wave; i < i1; i += kWaves) {
        const int tile_bytes = (i - i0) * LL::kTileBytes;
        LDS_PTR(float) rows = s_lds + (i - i0) * 16 * W;
        f32x4 o[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) p[r] = score_at(rows, n, 16 * vb + 4 * g + r - shift - n + L, W);
            const u32x2 pb = {Mma<DT>::pack(p[0], p[1]), Mma<DT>::pack(p[2], p[3])};
            LDS_PTR(char) blk = v_lds + tile_bytes + vb * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) o[ct] = Mma<DT>::k16(read_tr(blk + v_lane.off[ct]), pb, o[ct]);
        }
        const int qrow = 16 * i + n;
        u32x2 ow[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) ow[ct] = pack_acc<DT>(o[ct], 1.f);
        store_tile<C>(os, qrow * pitch, ow, g, stores_whole_lines(pitch, C, 0), pitch);
    }
}

template <int C> constexpr bool gather_exact_regions() { return C == 16; }

// =============================================================================
// P3: out[b,u,c] = sum_j attn[b,u+L-j,j] * x[b,u+L-j,c]
// =============================================================================
template <class DT, int C, int NBV>
__global__ void __launch_bounds__(kThreads)
gather_kernel(char *__restrict__ out, const float *__restrict__ attn, const char *__restrict__ x, uint32_t items,
              int T, int W, int L, int tiles, int nt, int strips, uint32_t strips_magic, int shift, int pitch) {
    using LL = Lds<C>;
    constexpr int CT = C / 16;
    constexpr int MT = kBandMaxTiles;
    fetch_args_now(out, attn, x, items, T, W, L, tiles, nt, strips, strips_magic, shift, pitch);
    // Key block kp (rows 16*kp - shift ...) is virtual block vb of query tile kp - vb, so the blocks that touch the
    // strip's rows need the query tiles i0 - hb .. i1 - 1 + ha.  Dynamic LDS: their x rows (qtiles tiles) and their
    // score rows (qtiles*16 x W fp32); at 16 channels, where a tile is half a copy chunk and the padding of the two
    // regions is what stands between seven and eight workgroups on a CU, neither is padded to whole chunks
    // (stage_exact; wider heads gain no workgroup by it and lose 1-2 % to the shorter last copy)
    constexpr bool kExact = gather_exact_regions<C>();
    const int hb = NBV - 1 - (shift >> 4), ha = (shift + 15) >> 4, qtiles = nt + hb + ha;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    LDS_PTR(char) x_lds = (LDS_PTR(char))smem;
    LDS_PTR(float) s_lds = (LDS_PTR(float))(x_lds + (kExact ? qtiles * LL::kTileBytes : region_bytes<C>(qtiles)));

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t item = xcd_item(blockIdx.x, items);
    const uint32_t b = div_by(item, strips, strips_magic);
    const int strip = (int)(item - b * strips);
    const int i0 = strip * nt, i1 = min(i0 + nt, tiles);
    const int g = lane >> 4, n = lane & 15;
    const int q0 = i0 - hb;                                            // first query tile needed

    const int64_t seq_off = (int64_t)b * T * pitch;      // packed rows of head_dim = pitch / 2 channels
    {
        const int rows_hi = min(T, 16 * (q0 + qtiles));
        const int lane_off = direct_lane_offset<C>(wave, lane, pitch, pitch);
        const Rsrc xs = make_rsrc(x + seq_off, rows_hi * pitch), ss = make_rsrc(attn + (int64_t)b * T * W, rows_hi * W * 4);
        constexpr int kRowRounds = (region_bytes<C>(MT + NBV) / kChunk + kWaves - 1) / kWaves;
        constexpr int kScoreRounds = (((kBandMaxTiles + NBV) * 16 * (16 * NBV - 15) * 4 + kChunk - 1) / kChunk + kWaves - 1) / kWaves;
        const int x_first = 16 * q0 * pitch + lane_off, x_step = (kChunk / LL::kRowBytes) * pitch;
        const int s_first = 16 * q0 * W * 4 + lane * 16;
        auto x_at = [&](int c) { return x_first + c * x_step; };
        auto s_at = [&](int c) { return s_first + c * kChunk; };
        if constexpr (kExact) {
            if (strips == 1) {      // nobody else reads these rows
                stage_exact<kReadOnce, kRowRounds>(xs, x_lds, qtiles * LL::kTileBytes, wave, lane, x_at);
                stage_exact<kReadOnce, kScoreRounds>(ss, (LDS_PTR(char))s_lds, qtiles * 16 * W * 4, wave, lane, s_at);
            } else {
                stage_exact<kReadShared, kRowRounds>(xs, x_lds, qtiles * LL::kTileBytes, wave, lane, x_at);
                stage_exact<kReadShared, kScoreRounds>(ss, (LDS_PTR(char))s_lds, qtiles * 16 * W * 4, wave, lane, s_at);
            }
        } else if (strips == 1) {
            stage_direct<C, MT + NBV, kReadOnce>(xs, 16 * q0, x_lds, qtiles, wave, lane_off, pitch);
            stage_scores<NBV, kReadOnce>(ss, 16 * q0 * W, s_lds, qtiles, W, wave, lane);
        } else {
            stage_direct<C, MT + NBV, kReadShared>(xs, 16 * q0, x_lds, qtiles, wave, lane_off, pitch);
            stage_scores<NBV, kReadShared>(ss, 16 * q0 * W, s_lds, qtiles, W, wave, lane);
        }
    }
    TrLane<C> x_tr;
    x_tr.init(0, lane);
    const int row_lo = 16 * i0, row_hi = min(T, 16 * i1);            // rows this strip owns
    const Rsrc os = make_rsrc(out + seq_off + (int64_t)row_lo * pitch, (row_hi - row_lo) * pitch);
    wait_direct();
    __syncthreads();

    // key block kp covers rows 16*kp - shift .. +15 and is virtual block vb of query tile kp - vb; lane (n, g)
    // holds key row n of the block against queries 4g+r of that tile: slot j = 16*vb - shift + n - (4g+r) + L
    const int kp_lo = i0 + (shift >> 4), kp_hi = i1 - 1 + ha;
    for (int kp = kp_lo + wave; kp <= kp_hi; kp += kWaves) {
        f32x4 acc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int vb = 0; vb < NBV; ++vb) {
            const int tq = kp - vb - q0;                               // in [0, qtiles) by the choice of hb and ha
            LDS_PTR(float) rows = s_lds + tq * 16 * W;
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) p[r] = score_at(rows, 4 * g + r, 16 * vb - shift + n - (4 * g + r) + L, W);
            const u32x2 pb = {Mma<DT>::pack(p[0], p[1]), Mma<DT>::pack(p[2], p[3])};
            LDS_PTR(char) xt = x_lds + tq * LL::kTileBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) acc[ct] = Mma<DT>::k16(read_tr(xt + x_tr.off[ct]), pb, acc[ct]);
        }
        const int row_off = (16 * (kp - i0) - shift + n) * pitch;       // outside the strip -> dropped
        u32x2 ow[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) ow[ct] = pack_acc<DT>(acc[ct], 1.f);
        store_tile<C>(os, row_off, ow, g, stores_whole_lines(pitch, C, shift), pitch);
    }
}

// ----------------------------------------------------------------------------- launchers
constexpr size_t kLdsPerCu = 160 * 1024;

// Strip length: the cover's ceiling, shortened until the workgroup's LDS (a function of it) fits a CU.
template <class F>
inline int fit_tiles(int max_tiles, F lds_of) {
    int nt = max_tiles;
    while (nt >= 1 && lds_of(nt) > kLdsPerCu) --nt;
    return nt;
}

template <class DT, int C, int NBV>
int launch_qk_n(float *attn, const void *a, const void *b, const Geom &g, const BandCover &c, hipStream_t s) {
    auto lds_of = [&](int nt) {
        const int kt = nt - 1 + NBV + ((c.shift & 15) ? 1 : 0);
        const bool direct = qk_keys_direct<C, NBV>();
        return (size_t)(direct ? 0 : region_bytes<C>(kt)) + (size_t)kWaves * 32 * g.W * sizeof(float) +
               (!direct && qk_spare_words<C>(kt) ? 0 : 64 * sizeof(float));
    };
    const int mt = fit_tiles(c.max_tiles, lds_of);
    if (mt < 1) return NA1D_ERR_UNSUPPORTED;
    const Split sp = make_split(g.B, g.T, mt);
    if (sp.items > 0x7fffff00LL || !div_magic_ok(sp.items, sp.strips)) return NA1D_ERR_UNSUPPORTED;
    auto kern = qk_kernel<DT, C, NBV>;
    const size_t lds = lds_of(sp.nt);
    if (!allow_lds(kern, lds)) return NA1D_ERR_LAUNCH;
    note_kernel("qk_kernel", DT::tag, C, NBV);
    launch_kernel(kern, (unsigned)sp.items, lds, s, attn, (const char *)a, (const char *)b, (uint32_t)sp.items, (int)g.T,
                                                   g.W, g.L, sp.tiles, sp.nt, sp.strips, div_magic(sp.strips), c.shift, 2 * g.C);
    return launch_status();
}

template <class DT, int C, int NBV>
int launch_av_n(void *out, const float *attn, const void *v, const Geom &g, const BandCover &c, hipStream_t s) {
    auto lds_of = [&](int nt) {
        return (size_t)region_bytes<C>(nt - 1 + NBV + ((c.shift & 15) ? 1 : 0)) + score_bytes(nt, g.W);
    };
    const int mt = fit_tiles(c.max_tiles, lds_of);
    if (mt < 1) return NA1D_ERR_UNSUPPORTED;
    const Split sp = make_split(g.B, g.T, mt);
    if (sp.items > 0x7fffff00LL || !div_magic_ok(sp.items, sp.strips)) return NA1D_ERR_UNSUPPORTED;
    auto kern = av_kernel<DT, C, NBV>;
    const size_t lds = lds_of(sp.nt);
    if (!allow_lds(kern, lds)) return NA1D_ERR_LAUNCH;
    note_kernel("av_kernel", DT::tag, C, NBV);
    launch_kernel(kern, (unsigned)sp.items, lds, s, (char *)out, attn, (const char *)v, (uint32_t)sp.items, (int)g.T, g.W,
                                                   g.L, sp.tiles, sp.nt, sp.strips, div_magic(sp.strips), c.shift, 2 * g.C);
    return launch_status();
}

template <class DT, int C, int NBV>
int launch_gather_n(void *out, const float *attn, const void *x, const Geom &g, const BandCover &c, hipStream_t s) {
    const int halo = NBV - 1 - (c.shift >> 4) + ((c.shift + 15) >> 4);          // query tiles beyond the strip
    auto lds_of = [&](int nt) {
        return gather_exact_regions<C>() ? (size_t)(nt + halo) * Lds<C>::kTileBytes + (size_t)(nt + halo) * 16 * g.W * 4
                                         : (size_t)region_bytes<C>(nt + halo) + score_bytes(nt + halo, g.W);
    };
    const int mt = fit_tiles(c.max_tiles, lds_of);
    if (mt < 1) return NA1D_ERR_UNSUPPORTED;
    const Split sp = make_split(g.B, g.T, mt);
    if (sp.items > 0x7fffff00LL || !div_magic_ok(sp.items, sp.strips)) return NA1D_ERR_UNSUPPORTED;
    auto kern = gather_kernel<DT, C, NBV>;
    const size_t lds = lds_of(sp.nt);
    if (!allow_lds(kern, lds)) return NA1D_ERR_LAUNCH;
    note_kernel("gather_kernel", DT::tag, C, NBV);
    launch_kernel(kern, (unsigned)sp.items, lds, s, (char *)out, attn, (const char *)x, (uint32_t)sp.items, (int)g.T, g.W,
                                                   g.L, sp.tiles, sp.nt, sp.strips, div_magic(sp.strips), c.shift, 2 * g.C);
    return launch_status();
}

#define NA1D_BAND_BLOCKS(FN, ...)                          \
    do {                                                   \
        const BandCover c = band_cover(g);                 \
        switch (c.nbv) {                                   \
            case 2: return FN<DT, C, 2>(__VA_ARGS__, c, s); \
            case 3: return FN<DT, C, 3>(__VA_ARGS__, c, s); \
            case 4: return FN<DT, C, 4>(__VA_ARGS__, c, s); \
            case 5: return FN<DT, C, 5>(__VA_ARGS__, c, s); \
            case 6: return FN<DT, C, 6>(__VA_ARGS__, c, s); \
        }                                                  \
        return NA1D_ERR_UNSUPPORTED;                       \
    } while (0)

template <class DT, int C>
int launch_qk(float *attn, const void *a, const void *b, const Geom &g, hipStream_t s) {
    NA1D_BAND_BLOCKS(launch_qk_n, attn, a, b, g);
}
template <class DT, int C>
int launch_av(void *out, const float *attn, const void *v, const Geom &g, hipStream_t s) {
    NA1D_BAND_BLOCKS(launch_av_n, out, attn, v, g);
}
template <class DT, int C>
int launch_gather(void *out, const float *attn, const void *x, const Geom &g, hipStream_t s) {
    NA1D_BAND_BLOCKS(launch_gather_n, out, attn, x, g);
}

int qk(float *attn, const void *a, const void *b, const Geom &g, int dtype, hipStream_t s) {
    if (!band_cover(g).nbv) return NA1D_ERR_UNSUPPORTED;
    NA1D_MFMA_DISPATCH(launch_qk, attn, a, b, g, s);
}
int av(void *out, const float *attn, const void *v, const Geom &g, int dtype, hipStream_t s) {
    if (!band_cover(g).nbv) return NA1D_ERR_UNSUPPORTED;
    NA1D_MFMA_DISPATCH(launch_av, out, attn, v, g, s);
}
int gather(void *out, const float *attn, const void *x, const Geom &g, int dtype, hipStream_t s) {
    if (!band_cover(g).nbv) return NA1D_ERR_UNSUPPORTED;
    NA1D_MFMA_DISPATCH(launch_gather, out, attn, x, g, s);
}

}  // namespace mfma
}  // namespace na1d
