// Shared machinery of the MFMA (matrix-core) NA1D kernels for gfx950.
//
// Tiles.  A sequence is cut into 16-row tiles at multiples of 16.  A query tile
// (rows t0 .. t0+15) meets keys t0-L .. t0+15+R, 15+W rows, which are covered by
// NBV "virtual" key blocks of 16 consecutive rows starting at row t0 - shift:
//   NBV = 2 (W <= 17): shift = L, the 32 rows start exactly at the first key;
//   NBV = 3 (L, R <= 16, W <= 32): shift = 16.
// The band product is then NBV 16x16 MFMA tiles
//
//   S^T[key, query] = K_blk (A: 16 keys x C) . Q_tile^T (B: C x 16 queries)
//
// The accumulator of v_mfma_f32_16x16x16 puts element (row 4g+r, col n) in lane
// 16g+n, register r (g = lane/16, n = lane%16).  For S^T that is "query n, keys
// 4g..4g+3": per-query quantities (row max, row sum, LSE) are lane-local up to a
// reduction over g, and the same registers, rounded to 16 bit, are exactly the B
// operand (k = key) of
//
//   O^T[chan, query] = V_blk^T (A: 16 chans x 16 keys) . P^T (B: 16 keys x 16 queries)
//
// so probabilities never leave registers.  V^T (and every other operand whose
// contraction index runs along memory rows) comes from LDS through
// ds_read_b64_tr_b16, which hands lane n of a 16-lane group column n of a 4x16
// tile of 16-bit values whose rows the group's lanes addressed four lanes apiece.
//
// Lane (n, g) holds, for query n, virtual keys 16*vb + 4g + r, i.e. window slot
// j = 16*vb + 4g + r - shift - n + L.  With three blocks and W <= 32 a lane never
// needs block 0 and block 2 in the same register r (block 0 is in the band only
// for 4g+r-n >= 16-L, block 2 only for 4g+r-n <= R-16), so the two are merged
// into one set of four slots: every lane carries 8 score slots either way.
//
// Work.  A workgroup of four waves owns a strip of up to kMaxTiles<C> consecutive
// tiles of one sequence.  It first copies the strip's rows of every operand
// (plus one 16-row halo block each side for the key-side operands) into LDS with
// all loads in flight at once - buffer loads that write LDS directly, so rows
// outside the sequence arrive as zeros, which is the band's zero fill - then, after
// one barrier, each wave computes tiles wave, wave+4, ... entirely out of LDS.
#pragma once

#include <algorithm>
#include <cstdio>
#include <type_traits>

#include <hip/hip_ext.h>

#include "na1d_common.h"

namespace na1d {
namespace mfma {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define LDS_PTR(T) __attribute__((address_space(3))) T *

constexpr int kWaves = 4;            // waves per workgroup
constexpr int kThreads = 64 * kWaves;
constexpr float kNegInf = -__builtin_inff();

// ---- per-dtype MFMA wrappers; operands travel as raw 32-bit registers --------
template <class DT> struct Mma;
template <> struct Mma<FP16> {
    __device__ static inline f32x4 k16(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
    }
    __device__ static inline f32x4 k32(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    __device__ static inline uint32_t pack(float lo, float hi) {
        f32x2 x = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
    }
};
template <> struct Mma<BF16> {
    __device__ static inline f32x4 k16(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(i16x4, a), __builtin_bit_cast(i16x4, b), c, 0, 0, 0);
    }
    __device__ static inline f32x4 k32(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    __device__ static inline uint32_t pack(float lo, float hi) {
        f32x2 x = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
    }
};

// ---- buffer resources -----------------------------------------------------------
// Raw buffer resource over one sequence of one tensor: loads outside [0, bytes)
// return zero and stores outside are dropped - no branches, no clamping.
using Rsrc = __amdgpu_buffer_rsrc_t;
__device__ inline Rsrc make_rsrc(const void *base, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// Cache policy of the streaming accesses (the `aux` operand of the buffer builtins; bit 1 = nt, non-temporal).
// Outputs are written once and rows that only one workgroup reads are read once: both are marked nt, which is
// worth 10-15 % of a forward launch here.  Rows that a neighbouring strip reads again as its halo are loaded
// with the default policy so that the second read hits L2 (marking them nt costs cfg2's forward 15 %).
constexpr int kReadOnce = 2, kReadShared = 0, kStoreAux = 2;
// A wave stores 16 rows of 2*C bytes starting `first_row` rows off a tile boundary.  The non-temporal policy
// pays only when the wave's rows make up whole 128-byte lines by themselves: packed rows starting on a line, or
// strided rows that are whole lines each.  Otherwise other waves (or other heads' workgroups) write the rest of
// the lines later, and only the default policy lets L2 merge the pieces.
__device__ inline bool stores_whole_lines(int pitch, int C, int first_row) {
    if (pitch == 2 * C) return (first_row * pitch) % 128 == 0 && (16 * pitch) % 128 == 0;
    return (2 * C) % 128 == 0 && pitch % 128 == 0;
}

// ---- LDS layout -------------------------------------------------------------------
// Rows of C 16-bit channels, row-major and unpadded; the 16-byte units of a row
// are XOR-swizzled with the row's 256-byte phase so that the 16 rows an operand
// read touches land in distinct banks.  The swizzle term repeats every 16 rows.
template <int C> struct Lds {
    static constexpr int kUnits = C / 8;                 // 16-byte units per row
    static constexpr int kRowBytes = 2 * C;
    static constexpr int kTileBytes = 16 * kRowBytes;
    static constexpr int kRowsPerPhase = kUnits >= 16 ? 1 : 16 / kUnits;   // rows per 256 bytes
    __device__ static inline int swz(int row) { return (int)((uint32_t)row / kRowsPerPhase) & (kUnits - 1); }     // row >= 0
    // byte address of (row, byte-in-row)
    __device__ static inline int addr(int row, int byte) {
        return row * kRowBytes + ((((byte >> 4) ^ swz(row)) << 4) | (byte & 15));
    }
};

// Tiles per strip (compile-time ceiling that sizes LDS and the copy loops).
template <int C> struct Strip {
    static constexpr int kMaxTiles = C <= 32 ? 8 : C <= 64 ? 4 : 2;
};

// Copy up to NTILES tiles of rows, starting at row_lo of a sequence, into an LDS
// region with buffer loads that write LDS directly: no registers are held while the
// loads are in flight.  NTILES fixes the (unrolled) number of loads per wave; the
// caller's buffer resource ends where the wanted rows end.  One wave's
// load fills 1 KB of consecutive LDS (lane l -> bytes 16l .. 16l+15 behind the
// wave-uniform base), so each lane asks for the 16-byte unit that belongs at that
// place under the XOR swizzle.  Chunk c of a region is loaded by wave c % kWaves; the
// swizzle repeats every four chunks at most, so a lane's offset inside its chunk is
// one constant.  Regions are padded to whole chunks (region_bytes); rows outside the
// resource arrive as zeros.  The loads count on vmcnt: wait for them before the
// workgroup barrier that publishes the regions.
constexpr int kChunk = 1024;
static_assert(kWaves % 4 == 0, "chunk -> swizzle phase mapping assumes a multiple of four waves");
template <int C> constexpr int region_bytes(int ntiles) {      // unsigned: a shift and a mask where the count is a run-time value
    return (int)(((uint32_t)(ntiles * Lds<C>::kTileBytes) + kChunk - 1) / kChunk * kChunk);
}
// `pitch` is the distance in bytes between consecutive rows in memory, `width` the bytes of a row that exist
// there (2 * head_dim; both 2*C when the rows are packed and as wide as the kernel's C).  A head_dim below C is
// zero-padded on the way in: the units past `width` ask for an address no resource reaches, and arrive as zeros.
constexpr int kNowhere = 0x60000000;     // beyond any resource (they end below 2^30), whatever small offset is added
template <int C>
__device__ inline int direct_lane_offset(int wave, int lane, int pitch = Lds<C>::kRowBytes, int width = Lds<C>::kRowBytes) {
    const int u = wave * 64 + lane;      // 16-byte unit inside chunks wave, wave + 4, ...
    const int su = u % Lds<C>::kUnits;
    const int unit = su ^ Lds<C>::swz(u / Lds<C>::kUnits);
    return unit * 16 < width ? (lane / Lds<C>::kUnits) * pitch + unit * 16 : kNowhere;
}
// One wave-wide load that writes LDS directly: lane l's BYTES (4 or 16) land at lds + BYTES * l.  Written out by hand
// so that the compiler knows nothing of it: told of such loads it puts a wait for ALL loads in flight in front of every
// LDS read it cannot tell apart from their target (the bias table, for one), and so serialises what was issued early
// on purpose.  Callers wait with wait_direct() before they (or, behind a barrier, other waves) read the target.
template <int BYTES, int AUX>
__device__ inline void load_to_lds(Rsrc src, LDS_PTR(char) lds, int offset) {
    static_assert((BYTES == 4 || BYTES == 16) && (AUX == 0 || AUX == 1 || AUX == 2 || AUX == 3), "load size / cache policy");
    const uint32_t at = __builtin_amdgcn_readfirstlane((uint32_t)reinterpret_cast<uintptr_t>(lds));      // wave-uniform by contract
    if constexpr (BYTES == 16) {
        if constexpr (AUX == 0) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(at), "v"(offset), "s"(src) : "memory");
        if constexpr (AUX == 1) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen sc0 lds" ::"s"(at), "v"(offset), "s"(src) : "memory");
        if constexpr (AUX == 2) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds" ::"s"(at), "v"(offset), "s"(src) : "memory");
        if constexpr (AUX == 3) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen sc0 nt lds" ::"s"(at), "v"(offset), "s"(src) : "memory");
    } else {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" ::"s"(at), "v"(offset), "s"(src) : "memory");
    }
}

template <int C, int NTILES, int AUX, int NW = kWaves>       // NW: the waves of the workgroup that share the copy
__device__ inline void stage_direct(Rsrc src, int row_lo, LDS_PTR(char) region, int ntiles, int wave, int lane_off,
                                    int pitch = Lds<C>::kRowBytes) {
    static_assert(NW % 4 == 0, "chunk -> swizzle phase mapping assumes a multiple of four waves");
    constexpr int kRounds = (region_bytes<C>(NTILES) / kChunk + NW - 1) / NW;
    constexpr int kChunkRows = kChunk / Lds<C>::kRowBytes;
    const int chunks = (int)((uint32_t)region_bytes<C>(ntiles) / kChunk);
    const int base = row_lo * pitch + lane_off, step = kChunkRows * pitch;
#pragma unroll
    for (int j = 0; j < kRounds; ++j) {
        const int c = j * NW + wave;
        if (c < chunks) load_to_lds<16, AUX>(src, region + c * kChunk, base + c * step);
    }
}
// The same into a region of exactly `bytes` bytes (a multiple of 16) that is not padded to whole chunks: the last chunk
// is loaded by as many lanes as it has 16-byte units, so nothing is written behind the region and another region can
// follow it directly.  LDS is granted in units of 1280 bytes; the kilobyte or so of padding that two regions carry can
// be the difference between seven and eight workgroups on a CU.
template <int AUX, int ROUNDS, int NW = kWaves, class OFFSET>
__device__ inline void stage_exact(Rsrc src, LDS_PTR(char) region, int bytes, int wave, int lane, OFFSET offset_of_chunk) {
    const int whole = bytes / kChunk, tail = bytes - whole * kChunk;
#pragma unroll
    for (int j = 0; j < ROUNDS; ++j) {
        const int c = j * NW + wave;
        if (c < whole) {
            load_to_lds<16, AUX>(src, region + c * kChunk, offset_of_chunk(c));
        } else if (c == whole && lane * 16 < tail) {       // only these lanes take part: the others' units do not exist
            load_to_lds<16, AUX>(src, region + c * kChunk, offset_of_chunk(c));
        }
    }
}
// The same for packed rows (pitch = width = 2*C bytes) into a region of NTILES tiles, all of it: how many chunks there
// are, which of them a wave loads and where they go is then known at compile time, and a copy is an add for M0 and the
// load (rows past the resource's end are asked for all the same; they cost an instruction, no traffic).
template <int C, int NTILES, int AUX, int NW = kWaves>
__device__ inline void stage_packed(Rsrc src, int row_lo, LDS_PTR(char) region, int wave, int lane_off) {
    static_assert(NW % 4 == 0, "chunk -> swizzle phase mapping assumes a multiple of four waves");
    constexpr int kChunks = region_bytes<C>(NTILES) / kChunk, kRounds = (kChunks + NW - 1) / NW;
    const int base = row_lo * Lds<C>::kRowBytes + lane_off + wave * kChunk;     // a chunk of packed rows is a chunk of memory
    LDS_PTR(char) mine = region + wave * kChunk;
#pragma unroll
    for (int j = 0; j < kRounds; ++j)
        if ((j + 1) * NW <= kChunks || wave < kChunks - j * NW) load_to_lds<16, AUX>(src, mine + j * NW * kChunk, base + j * NW * kChunk);
}
__device__ inline void wait_direct() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// Workgroup barrier that waits for this wave's LDS accesses only.  __syncthreads() also waits for every vector-memory
// access in flight, i.e. for strip copies that were issued early on purpose; what has to have landed is waited for
// explicitly (wait_direct) in front of this.
__device__ inline void barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// Have a value worked out here rather than where it is first used: per-lane constants placed in front of the wait for
// the strip copies cost nothing, behind it they delay the first tile.
template <class T> __device__ inline void settle(T &x) { asm volatile("" : "+v"(x)); }

// ---- operands out of LDS ------------------------------------------------------
// Row operand (A or B of a contraction over channels): lane (n, g) holds row n of a
// 16-row tile; a 32-wide step s covers channels 32s + 8g .. +7, the 16-wide
// remainder channels 32*k32 + 4g .. +3.  Offsets are per-lane constants.
template <int C> struct RowOperand {
    static constexpr int k32 = C / 32;
    static constexpr int k16 = (C % 32) / 16;
    u32x4 w32[k32 > 0 ? k32 : 1];
    u32x2 w16[k16 > 0 ? k16 : 1];
};
// CS is the width in channels of the rows as they are staged: C, or several heads of C channels side by side, in
// which case `sub` is the byte offset of this lane's head inside a staged row.
template <int C, int CS = C> struct RowLane {        // this lane's byte offsets for a row operand whose tile starts `row0` rows into a region
    int off32[RowOperand<C>::k32 > 0 ? RowOperand<C>::k32 : 1];
    int off16;
    __device__ inline void init(int row0, int lane, int sub = 0) {
        const int g = lane >> 4, n = lane & 15;
#pragma unroll
        for (int s = 0; s < RowOperand<C>::k32; ++s) off32[s] = Lds<CS>::addr(row0 + n, sub + 64 * s + 16 * g);
        off16 = Lds<CS>::addr(row0 + n, sub + 64 * RowOperand<C>::k32 + 8 * g);
    }
};
template <int C, int CS>
__device__ inline void read_rows(RowOperand<C> &o, LDS_PTR(char) tile, const RowLane<C, CS> &l) {
#pragma unroll
    for (int s = 0; s < RowOperand<C>::k32; ++s) o.w32[s] = *reinterpret_cast<LDS_PTR(u32x4)>(tile + l.off32[s]);
    if (RowOperand<C>::k16) o.w16[0] = *reinterpret_cast<LDS_PTR(u32x2)>(tile + l.off16);
}
// The same operand straight from memory, for rows that only this wave needs: lane (n, g) asks for its pieces of the
// row `n` rows behind byte offset `tile` of the resource (rows of `width` bytes, `pitch` bytes apart; pieces past the
// width, like rows past the resource's end, arrive as zeros).
template <int C, int AUX>
__device__ inline void load_rows(RowOperand<C> &o, Rsrc src, int tile, int pitch, int width, int lane) {
    const int g = lane >> 4, n = lane & 15;
    const int row = tile + n * pitch;
#pragma unroll
    for (int s = 0; s < RowOperand<C>::k32; ++s) {
        const int at = 64 * s + 16 * g;
        o.w32[s] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(src, at < width ? row + at : kNowhere, 0, AUX));
    }
    if (RowOperand<C>::k16) {
        const int at = 64 * RowOperand<C>::k32 + 8 * g;
        o.w16[0] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(src, at < width ? row + at : kNowhere, 0, AUX));
    }
}
template <class DT, int C>
__device__ inline f32x4 dot_rows_mma(const RowOperand<C> &a, const RowOperand<C> &b, f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f}) {
#pragma unroll
    for (int s = 0; s < RowOperand<C>::k32; ++s) acc = Mma<DT>::k32(a.w32[s], b.w32[s], acc);
    if (RowOperand<C>::k16) acc = Mma<DT>::k16(a.w16[0], b.w16[0], acc);
    return acc;
}

// Transposed operand: output lane (n, g) receives tile[row 4g+0..3][chan 16*ct + n];
// the lane supplies the address of row 4g + (n>>2), byte 32*ct + 8*(n&3).
template <int C, int CS = C> struct TrLane {
    int off[C / 16];
    __device__ inline void init(int row0, int lane, int sub = 0) {
        const int g = lane >> 4, n = lane & 15;
#pragma unroll
        for (int ct = 0; ct < C / 16; ++ct) off[ct] = Lds<CS>::addr(row0 + 4 * g + (n >> 2), sub + 32 * ct + 8 * (n & 3));
    }
};
__device__ inline u32x2 read_tr(LDS_PTR(char) p) {
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LDS_PTR(i16x4)>(p)));
}

// ---- reductions over g = lane/16 (lanes n, n+16, n+32, n+48), result in all four ----
// v_permlane16_swap / v_permlane32_swap exchange 16- and 32-lane rows between two
// registers, so swapping a value with itself lines up each lane's partner.
__device__ inline void swap_rows16(float x, float &a, float &b) {
    const u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    a = __uint_as_float(r.x);
    b = __uint_as_float(r.y);
}
__device__ inline void swap_rows32(float x, float &a, float &b) {
    const u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    a = __uint_as_float(r.x);
    b = __uint_as_float(r.y);
}
// Plain v_max_f32 / v_max3_f32: scores are never NaN, so the quieting that fmaxf()
// adds in front of every operand is skipped.
__device__ inline float max2(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ inline float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
// Maximum of eight values that may come straight out of matrix-core accumulators.  The compiler keeps the wait
// states between a matrix instruction and a vector instruction that reads its result, but it cannot see into inline
// assembly, so the block brings its own: up to 11 idle states are owed after the widest product used here (16x16x32).
__device__ inline float max8_of_accumulators(const float (&x)[4], const float (&y)[4]) {
    float a, b, c;
    asm("s_nop 7\n\ts_nop 3\n\t"
        "v_max3_f32 %0, %3, %4, %5\n\tv_max3_f32 %1, %6, %7, %8\n\tv_max_f32 %2, %9, %10\n\tv_max3_f32 %0, %0, %1, %2"
        : "=&v"(a), "=&v"(b), "=&v"(c)
        : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(y[0]), "v"(y[1]), "v"(y[2]), "v"(y[3]));
    return a;
}
__device__ inline float xor_max(float x) {
    float a, b;
    swap_rows16(x, a, b);
    swap_rows32(max2(a, b), a, b);
    return max2(a, b);
}
__device__ inline float xor_sum(float x) {
    float a, b;
    swap_rows16(x, a, b);
    swap_rows32(a + b, a, b);
    return a + b;
}

// ---- tile stores -------------------------------------------------------------------
// Pack an accumulator (lane (n, g): row n, channels 16*ct + 4g .. 4g+3) times `f` into four 16-bit values.
template <class DT> __device__ inline u32x2 pack_acc(f32x4 a, float f) {
    return u32x2{Mma<DT>::pack(a[0] * f, a[1] * f), Mma<DT>::pack(a[2] * f, a[3] * f)};
}
// Store a 16 x C tile held as one u32x2 per channel tile.  Channel tiles are paired so that a lane writes 16
// contiguous bytes: v_permlane16_swap hands lanes of even g the neighbour's half of the even tile and lanes of odd
// g the neighbour's half of the odd tile.  Half as many stores, and one instruction writes whole 64-byte pieces of
// a row instead of 32-byte halves that the other instruction completes later.
template <int C, int AUX>
__device__ inline void store_tile(Rsrc dst, int row_byte, const u32x2 (&w)[C / 16], int g, int width) {
    constexpr int CT = C / 16;
    if constexpr (CT == 1) {
        __builtin_amdgcn_raw_buffer_store_b64(w[0], dst, g * 8 < width ? row_byte + g * 8 : kNowhere, 0, AUX);
    } else {
#pragma unroll
        for (int p = 0; p < CT / 2; ++p) {
            const u32x2 lo = __builtin_amdgcn_permlane16_swap(w[2 * p].x, w[2 * p + 1].x, false, false);
            const u32x2 hi = __builtin_amdgcn_permlane16_swap(w[2 * p].y, w[2 * p + 1].y, false, false);
            const u32x4 v = {lo.x, hi.x, lo.y, hi.y};
            const int at = (2 * p + (g & 1)) * 32 + (g >> 1) * 16;      // channels past head_dim are not stored
            __builtin_amdgcn_raw_buffer_store_b128(v, dst, at < width ? row_byte + at : kNowhere, 0, AUX);
        }
    }
}
template <int C>
__device__ inline void store_tile(Rsrc dst, int row_byte, const u32x2 (&w)[C / 16], int g, bool stream, int width) {
    if (stream)
        store_tile<C, kStoreAux>(dst, row_byte, w, g, width);
    else
        store_tile<C, 0>(dst, row_byte, w, g, width);
}

// ---- window slots of a lane ------------------------------------------------------
template <int NBV> struct Window {
    // slot sets: X = block 0 (NBV 2) or merged blocks 0/2 (NBV 3);  Y = block 1
    float bias_x[4], bias_y[4];   // log2-domain rpb, -inf outside the band
    bool from0[4];                // NBV 3: slot r of X comes from block 0 (else block 2)
    u32x2 keep0, keep2;           // NBV 3: 16-bit lane masks that split packed X into blocks 0 and 2
};

// Window slots and bias of a lane, by way of a small table in LDS.  Every wave writes the table of its head
// itself - entry i holds the log2-domain bias of window slot j = i - kBiasPad, or -inf where j lies outside
// [0, W) - with a tiny load issued BEFORE the strip copies (it hits L2; a NULL rpb makes an empty resource, which
// reads as zeros), and each lane then picks its eight entries with plain LDS reads: no compares, selects or
// multiply-adds per slot, which for short sequences were a large share of a wave's vector instructions.  Waves
// that work on the same head share one table: they write the same values, and a wave reads after its own writes.
constexpr int kBiasPad = 32, kBiasEntries = 64;         // slots -32 .. 31 cover every block's reach (W <= 32)
struct BiasTable {
    float raw;
};
// The load is written out by hand: the compiler, which cannot count the strip copies that follow it through their
// branches, would otherwise put a wait for ALL of them in front of the value's first use.  The caller waits instead:
// wait_bias() behind any wait that covers the loads issued up to here (loads return in the order they were issued).
__device__ inline void load_bias_table(BiasTable &t, const float *rpb_h, int W, int lane) {
    const uint64_t p = reinterpret_cast<uint64_t>(rpb_h);
    const u32x4 rs = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, p ? (uint32_t)W * 4u : 0u, 0x00020000u};   // NULL: empty, reads as zeros
    const int off = (lane - kBiasPad) * 4;                                                                         // outside [0, W): 0
    asm volatile("buffer_load_dword %0, %1, %2, 0 offen" : "=v"(t.raw) : "v"(off), "s"(rs) : "memory");
}
// Ties the value to the wait in front of it, so that nothing that uses it is moved ahead of that wait.
__device__ inline void wait_bias(BiasTable &t) { asm volatile("" : "+v"(t.raw) :: "memory"); }
__device__ inline void write_bias_table(LDS_PTR(float) tab, const BiasTable &t, int W, int lane, float mult = kLog2e) {
    tab[lane] = (uint32_t)(lane - kBiasPad) < (uint32_t)W ? t.raw * mult : kNegInf;
}
// The lane's slots out of the wave's own table (written by this wave: program order is enough).
template <int NBV>
__device__ inline void read_window(Window<NBV> &w, LDS_PTR(float) tab, int L, int shift, int g, int n) {
    const int j0 = 4 * g - n + L - shift;               // window slot of register 0 of block 0
    uint32_t m[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        w.from0[r] = NBV == 2 || j0 + r >= 0;
        const int jx = NBV == 3 ? ((j0 + r) & 31) : j0 + r;      // three blocks: block 2's slot where block 0 has none
        w.bias_x[r] = tab[jx + kBiasPad];
        w.bias_y[r] = tab[j0 + r + 16 + kBiasPad];
        m[r] = w.from0[r] ? 0xffffu : 0u;
    }
    w.keep0 = u32x2{m[0] | (m[1] << 16), m[2] | (m[3] << 16)};
    w.keep2 = u32x2{~w.keep0.x, ~w.keep0.y};
}

// ---- the model's additive mask on edge tiles --------------------------------------------
// A score gets the reference's -100 when its key lies outside [0, tv) and its query row is a valid one; a padded
// query row (row >= tv) has all of its slots masked there, a uniform shift that the softmax does not see, so it gets
// none here.  That makes the mask a product a[key] * b[query] - a = 1 on keys outside the range, b = -100 / scale on
// valid rows - and the matrix core adds it to a block's scores with one more instruction per block: a sits in
// channels 0 and 1 of a 16-channel operand, b as a 16-bit value and the rounding error of that value in the same two
// channels (their sum is -100 / scale to 2^-16).  Three vector instructions per block instead of four per score slot.
struct EdgeMask {
    uint32_t hi_lo;      // b's two channels, packed; 0 in the lanes that hold other channels (g != 0)
    uint32_t one2;       // two ones in the operand's type
};
template <class DT> __device__ inline EdgeMask make_edge_mask(float mask_x, int g) {
    // a half-precision operand cannot hold less than -65504: scales below 100 / 65504 get the largest mask it can
    const float m = DT::tag == NA1D_FP16 ? __builtin_fmaxf(mask_x, -60000.f) : mask_x;
    const uint32_t hi = Mma<DT>::pack(m, 0.f) & 0xffffu;
    const float hi_f = DT::tag == NA1D_BF16 ? __uint_as_float(hi << 16) : (float)__builtin_bit_cast(_Float16, (uint16_t)hi);
    const uint32_t lo = Mma<DT>::pack(m - hi_f, 0.f) & 0xffffu;
    return EdgeMask{g == 0 ? (hi | (lo << 16)) : 0u, DT::tag == NA1D_BF16 ? 0x3f803f80u : 0x3c003c00u};
}
// s[vb] += mask for the NBV key blocks of a tile whose first key row is key0 - n (key0 = that row + this lane's n).
template <class DT, int NBV>
__device__ inline void add_edge_mask(f32x4 (&s)[NBV], const EdgeMask &e, int key0, int qrow, int tv) {
    const u32x2 b = {qrow < tv ? e.hi_lo : 0u, 0u};
    uint32_t a[NBV];
#pragma unroll
    for (int vb = 0; vb < NBV; ++vb) {
        a[vb] = (uint32_t)(key0 + 16 * vb) >= (uint32_t)tv ? e.one2 : 0u;      // unsigned: also key < 0
        settle(a[vb]);
    }
#pragma unroll
    for (int vb = 0; vb < NBV; ++vb) s[vb] = Mma<DT>::k16(u32x2{a[vb], 0u}, b, s[vb]);
}

// A wave-uniform int32 through the scalar cache: it does not count on the vector-memory counter, so waiting for it
// does not wait for the strip copies in flight.
__device__ inline int load_uniform_i32(const int32_t *p, uint32_t index) {
    const int32_t *a = p + index;
    int v;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(a) : "memory");
    return v;
}

// Kernel arguments live in memory and the compiler fetches each one next to its
// first use, which here puts a scalar-load round trip in front of every region's
// copy.  Naming them in an empty asm at kernel entry makes all the fetches go out
// together, behind one wait.
template <class... A> __device__ inline void fetch_args_now(A... a) {
    ((void)0, ..., [](auto x) { asm volatile("" ::"s"(x)); }(a));
}

// ---- work split ---------------------------------------------------------------
// Division of a wave-uniform number by a launch constant d as one multiply-high:
// with m = floor(2^32 / d) + 1 the quotient is exact whenever n * d < 2^32.
inline uint32_t div_magic(int64_t d) { return d > 1 ? (uint32_t)((1ull << 32) / (uint64_t)d) + 1u : 0u; }
inline bool div_magic_ok(int64_t n_max, int64_t d) { return n_max < (1ll << 32) / d; }
__device__ inline uint32_t div_by(uint32_t n, int d, uint32_t magic) { return d == 1 ? n : __umulhi(n, magic); }

struct Split {
    int tiles;       // 16-row tiles per sequence
    int nt;          // tiles per strip
    int strips;      // strips per sequence
    int64_t items;   // workgroups
};
inline Split make_split(int64_t B, int64_t T, int max_tiles, int min_items = 1024) {
    Split s;
    s.tiles = (int)((T + 15) / 16);
    s.strips = (s.tiles + max_tiles - 1) / max_tiles;
    // small problems: more, shorter strips so that every CU gets a few workgroups (the backward, whose strips carry
    // a halo of query tiles, is better off with one workgroup per CU and longer strips)
    while (B * s.strips < min_items && s.strips < s.tiles) ++s.strips;
    s.nt = (s.tiles + s.strips - 1) / s.strips;
    s.strips = (s.tiles + s.nt - 1) / s.nt;
    s.items = B * s.strips;
    return s;
}

// Byte strides of one tensor family as the kernels take them.
struct Strides {
    int64_t sample, head;   // from one sample / head to the next
    int pitch;              // from one row to the next
    int width;              // bytes of a row that exist: 2 * head_dim
};
inline Strides byte_strides(const Layout &l, const Geom &g) {
    return Strides{2 * l.sample, 2 * l.head, (int)(2 * l.row), 2 * g.C};
}
// Offsets inside one sequence are 32-bit: the rows of a sequence, plus the halo rows the copies ask for
// beyond its end, must span less than 2^30 bytes.
inline bool strides_ok(const Layout &l, const Geom &g) { return l.row >= g.C && g.T + 96 <= (1 << 29) / l.row; }
inline bool items_ok(const Split &sp, const Geom &g) {
    return sp.items <= 0x7fffff00LL && div_magic_ok(sp.items, g.H) && div_magic_ok(sp.items, sp.strips);
}

// Workgroup id -> (sample, head, strip).  Heads vary fastest, then strips: workgroups that run side by side
// touch the same rows of a head-interleaved tensor (and neighbouring strips, which share halo rows), and
// xcd_item() keeps such a run of ids on one XCD, i.e. behind one L2.
struct WorkItem {
    uint32_t sample, head, item;   // item = (sample * H + head) * strips + strip: the d rpb partial-sum row
    int strip;
};
__device__ inline uint32_t xcd_item(uint32_t wg, uint32_t items);
__device__ inline WorkItem work_item(uint32_t wg, uint32_t items, int strips, uint32_t strips_magic, int H,
                                     uint32_t heads_magic) {
    const uint32_t lin = xcd_item(wg, items);
    const uint32_t rest = div_by(lin, H, heads_magic);
    WorkItem w;
    w.head = lin - rest * H;
    w.sample = div_by(rest, strips, strips_magic);
    w.strip = (int)(rest - w.sample * strips);
    w.item = (w.sample * H + w.head) * strips + w.strip;
    return w;
}

// Workgroup id -> work item, so that consecutive items (neighbouring strips of a
// sequence, which share halo rows) run on the same XCD and hit the same L2: the
// hardware deals workgroup ids round-robin over the 8 XCDs.
__device__ inline uint32_t xcd_item(uint32_t wg, uint32_t items) {
    const uint32_t per = items / 8;          // items in the evenly dealt part
    if (wg >= per * 8) return wg;            // ragged tail keeps its id
    return (wg & 7) * per + (wg >> 3);
}

// ---- fixed-order reduction of the bias gradient ----------------------------------------
// With a workspace the backward kernels write one row of STRIDE floats per workgroup (its sums over the window
// slots) instead of adding them to d rpb with float atomics; this kernel, one workgroup per (head, slot), then folds
// the rows of a head in a fixed order.
constexpr int kPartialStride = 32;          // windows of the two/three-block kernels: W <= 32
constexpr int kWidePartialStride = 80;      // wide windows: W <= 80
template <int STRIDE>
__global__ void __launch_bounds__(128)
drpb_reduce_kernel(float *__restrict__ drpb, const float *__restrict__ partial, int N, int H, int strips, int W) {
    __shared__ float acc[128];
    const int h = blockIdx.x / W, j = blockIdx.x - h * W;
    const int rows = N * strips;                      // items of this head: (n, strip)
    float s = 0.f;
    for (int i = threadIdx.x; i < rows; i += 128) {
        const int n = i / strips, st = i - n * strips;
        s += partial[((size_t)(n * H + h) * strips + st) * STRIDE + j];
    }
    acc[threadIdx.x] = s;
    __syncthreads();
    for (int half = 64; half > 0; half >>= 1) {       // fixed tree: the result does not depend on timing
        if ((int)threadIdx.x < half) acc[threadIdx.x] += acc[threadIdx.x + half];
        __syncthreads();
    }
    if (threadIdx.x == 0) drpb[h * W + j] += acc[0];
}

// While profiling events are set, the launchers note which kernel they are about to launch, spelt as a profiler's
// kernel trace prints it without namespaces and arguments, e.g. fused_bwd_kernel<FP16, 32, 2, false>.
inline void note_kernel(const char *base, int dtype, int C, int nbv, int drop = -1, int hg = 0) {
    LaunchEvents &ev = launch_events();
    if (!ev.start && !ev.stop) return;
    const char *dt = dtype == NA1D_BF16 ? "BF16" : "FP16";
    if (drop < 0)
        snprintf(ev.kernel, sizeof ev.kernel, "%s<%s, %d, %d>", base, dt, C, nbv);
    else if (hg <= 0)
        snprintf(ev.kernel, sizeof ev.kernel, "%s<%s, %d, %d, %s>", base, dt, C, nbv, drop ? "true" : "false");
    else
        snprintf(ev.kernel, sizeof ev.kernel, "%s<%s, %d, %d, %s, %d>", base, dt, C, nbv, drop ? "true" : "false", hg);
}

// The same for kernels with other template arguments: the name is spelt out by the caller.
template <class... A> inline void note_kernel_as(const char *format, A... a) {
    LaunchEvents &ev = launch_events();
    if (ev.start || ev.stop) snprintf(ev.kernel, sizeof ev.kernel, format, a...);
}

// Launch, with the calling thread's profiling events around the kernel if it has set any.  An operator of several
// kernels gives the first one the start event and the last one the stop event (`span`: bit 0 = this launch records
// start, bit 1 = it records stop).
template <class K, class... Args>
inline void launch_kernel_span(int span, K kern, unsigned grid, unsigned block, size_t lds, hipStream_t s, Args... args) {
    LaunchEvents &ev = launch_events();
    if (ev.start || ev.stop) {
        // events recorded by the launch itself do not belong in a captured graph: refuse instead of recording them
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (ev.refused || hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
            ev.refused = true;      // also what follows a refused launch in the same call
            return;
        }
        hipExtLaunchKernelGGL(kern, dim3(grid), dim3(block), (uint32_t)lds, s, (span & 1) ? ev.start : nullptr,
                              (span & 2) ? ev.stop : nullptr, 0, args...);
    } else {
        kern<<<grid, block, lds, s>>>(args...);
    }
}
template <class K, class... Args>
inline void launch_kernel_block(K kern, unsigned grid, unsigned block, size_t lds, hipStream_t s, Args... args) {
    launch_kernel_span(3, kern, grid, block, lds, s, args...);
}
template <class K, class... Args>
inline void launch_kernel(K kern, unsigned grid, size_t lds, hipStream_t s, Args... args) {
    launch_kernel_block(kern, grid, (unsigned)kThreads, lds, s, args...);
}

// Dynamic LDS above 64 KB has to be allowed per kernel.
template <class K>
inline bool allow_lds(K kern, size_t bytes) {
    if (bytes <= 64 * 1024) return true;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)bytes) == hipSuccess;
}

// Number of virtual key blocks the kernels need, 0 if the shape is not covered.
inline int window_blocks(const Geom &g) {
    const int R = g.W - 1 - g.L;
    if (g.C > 128) return 0;               // head_dim is run at the next of 16, 32, 64, 128, zero-padded
    if (g.T > (1 << 29) / g.C) return 0;   // per-sequence byte offsets stay in 31 bits
    if (15 + g.W <= 32) return 2;
    if (g.L <= 16 && R <= 16 && g.W <= 32) return 3;
    return 0;
}

// Rows between the first virtual key block and its query tile.  Three blocks: 16.  Two blocks: anything in
// [L, 16 - R] covers the window; the first multiple of a 128-byte line's worth of rows is taken, so that key
// blocks (the units dK / dV are written in) and the key-side copies start on a line.
inline int window_shift(const Geom &g) {
    if (window_blocks(g) != 2) return 16;
    const int R = g.W - 1 - g.L, rows = std::max(1, 128 / (2 * g.C));
    const int s = (g.L + rows - 1) / rows * rows;
    return s <= 16 - R ? s : g.L;
}

// The kernels' C for a head_dim: the next of 16, 32, 64, 128 (0 above).
inline int padded_width(int head_dim) { return head_dim <= 16 ? 16 : head_dim <= 32 ? 32 : head_dim <= 64 ? 64 : head_dim <= 128 ? 128 : 0; }

#define NA1D_MFMA_DISPATCH(FN, ...)                                            \
    do {                                                                       \
        if (dtype == NA1D_BF16) {                                              \
            switch (padded_width(g.C)) {                                                     \
                case 16: return FN<BF16, 16>(__VA_ARGS__);                     \
                case 32: return FN<BF16, 32>(__VA_ARGS__);                     \
                case 64: return FN<BF16, 64>(__VA_ARGS__);                     \
                case 128: return FN<BF16, 128>(__VA_ARGS__);                   \
            }                                                                  \
        } else {                                                               \
            switch (padded_width(g.C)) {                                                     \
                case 16: return FN<FP16, 16>(__VA_ARGS__);                     \
                case 32: return FN<FP16, 32>(__VA_ARGS__);                     \
                case 64: return FN<FP16, 64>(__VA_ARGS__);                     \
                case 128: return FN<FP16, 128>(__VA_ARGS__);                   \
            }                                                                  \
        }                                                                      \
        return NA1D_ERR_UNSUPPORTED;                                           \
    } while (0)


}  // namespace mfma
}  // namespace na1d
