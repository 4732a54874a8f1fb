// MFMA (matrix-core) NA1D kernels for gfx950.
//
// Geometry shared by every kernel here.  A sequence is cut into 16-row blocks at
// multiples of 16; block i is both "query tile i" and "key block i".  With
// left <= 16 and right <= 16 a query tile only ever meets key blocks i-1, i, i+1,
// so the band product is three 16x16 MFMA tiles per query tile:
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
// so probabilities never leave registers.  V^T (and the other operands that need
// the contraction index to run along memory rows) come from LDS through
// ds_read_b64_tr_b16, which hands lane n of a 16-lane group column n of a 4x16
// tile of 16-bit values whose rows the group's lanes addressed four lanes apiece.
//
// Every wave works alone on a strip of consecutive tiles of one sequence, with a
// private LDS ring of K/V blocks: no workgroup barriers anywhere.
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

constexpr int kWaves = 4;            // waves per workgroup (each independent)
constexpr int kRing = 4;             // K/V blocks resident per wave
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

// ---- LDS block layout ---------------------------------------------------------
// A block is 16 rows of C 16-bit channels, row-major, with the row stride padded
// so that the 16 rows of an operand read fall in distinct banks.
template <int C> struct Blk {
    static constexpr int kRowBytes = 2 * C;
    static constexpr int kStride = kRowBytes + (C == 16 ? 8 : 16);   // bytes
    static constexpr int kBytes = 16 * kStride;
    static constexpr int kUnit = (C == 16) ? 8 : 16;                 // bytes per lane per copy step
    static constexpr int kUnitsPerRow = kRowBytes / kUnit;
    static constexpr int kSteps = 16 * kUnitsPerRow / 64;            // copy steps per block
    static_assert(16 * kUnitsPerRow % 64 == 0, "block must be a whole number of wave copies");
};

template <int C> struct BlockRegs {   // one block in flight from global memory
    u32x4 v[Blk<C>::kSteps];
};

// Issue the global loads of block `kb` (rows 16kb .. 16kb+15) of a sequence that
// starts at `seq`; rows outside [0, T) read as zero.
template <int C>
__device__ inline void load_block(BlockRegs<C> &r, const char *__restrict__ seq, int kb, int T, int lane) {
    using B = Blk<C>;
#pragma unroll
    for (int s = 0; s < B::kSteps; ++s) {
        const int unit = s * 64 + lane;
        const int row = 16 * kb + unit / B::kUnitsPerRow;
        const int col = unit % B::kUnitsPerRow;
        u32x4 x = {0u, 0u, 0u, 0u};
        if (row >= 0 && row < T) {
            const char *p = seq + (int64_t)row * B::kRowBytes + col * B::kUnit;
            if (B::kUnit == 8) {
                const u32x2 y = *reinterpret_cast<const u32x2 *>(p);
                x.x = y.x;
                x.y = y.y;
            } else {
                x = *reinterpret_cast<const u32x4 *>(p);
            }
        }
        r.v[s] = x;
    }
}

template <int C>
__device__ inline void store_block(const BlockRegs<C> &r, LDS_PTR(char) slot, int lane) {
    using B = Blk<C>;
#pragma unroll
    for (int s = 0; s < B::kSteps; ++s) {
        const int unit = s * 64 + lane;
        LDS_PTR(char) p = slot + (unit / B::kUnitsPerRow) * B::kStride + (unit % B::kUnitsPerRow) * B::kUnit;
        if (B::kUnit == 8) {
            u32x2 y = {r.v[s].x, r.v[s].y};
            *reinterpret_cast<LDS_PTR(u32x2)>(p) = y;
        } else {
            *reinterpret_cast<LDS_PTR(u32x4)>(p) = r.v[s];
        }
    }
}

// Transposed operand: for output lane (n = lane%16, g = lane/16) the four values
// blk[row 4g+0..3][chan 16*ct + n].
template <int C>
__device__ inline u32x2 read_tr(LDS_PTR(char) slot, int ct, int lane) {
    const int g = lane >> 4, i = lane & 15;
    LDS_PTR(char) p = slot + (4 * g + (i >> 2)) * Blk<C>::kStride + ct * 32 + (i & 3) * 8;
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LDS_PTR(i16x4)>(p)));
}

// Contraction over channels:  acc += X_blk[row n][:] . Y[col][:]  with X from an LDS
// block (A operand, row = lane%16) and Y held in registers in the same channel
// order (B operand).  Channel order: step s of a 32-wide step covers channels
// 32s + 8g .. +7; a 16-wide step covers 16s + 4g .. +3.
template <int C> struct RowOperand {          // one 16-row tile as an A or B operand over all of C
    static constexpr int k32 = C / 32;
    static constexpr int k16 = (C % 32) / 16;
    u32x4 w32[k32 > 0 ? k32 : 1];
    u32x2 w16[k16 > 0 ? k16 : 1];
};

template <int C>
__device__ inline void read_rows(RowOperand<C> &o, LDS_PTR(char) slot, int lane) {
    const int g = lane >> 4, n = lane & 15;
    LDS_PTR(char) row = slot + n * Blk<C>::kStride;
#pragma unroll
    for (int s = 0; s < RowOperand<C>::k32; ++s) o.w32[s] = *reinterpret_cast<LDS_PTR(u32x4)>(row + 64 * s + 16 * g);
    if (RowOperand<C>::k16) o.w16[0] = *reinterpret_cast<LDS_PTR(u32x2)>(row + 64 * RowOperand<C>::k32 + 8 * g);
}

// Same operand straight from global memory (rows outside [0,T) are zero).
template <int C>
__device__ inline void load_rows(RowOperand<C> &o, const char *__restrict__ seq, int tile, int T, int lane) {
    const int g = lane >> 4, n = lane & 15;
    const int row = 16 * tile + n;
    const bool ok = row >= 0 && row < T;
    const char *p = seq + (int64_t)row * (2 * C);
#pragma unroll
    for (int s = 0; s < RowOperand<C>::k32; ++s) {
        u32x4 x = {0u, 0u, 0u, 0u};
        if (ok) x = *reinterpret_cast<const u32x4 *>(p + 64 * s + 16 * g);
        o.w32[s] = x;
    }
    if (RowOperand<C>::k16) {
        u32x2 x = {0u, 0u};
        if (ok) x = *reinterpret_cast<const u32x2 *>(p + 64 * RowOperand<C>::k32 + 8 * g);
        o.w16[0] = x;
    }
}

template <class DT, int C>
__device__ inline f32x4 dot_rows_mma(const RowOperand<C> &a, const RowOperand<C> &b) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < RowOperand<C>::k32; ++s) acc = Mma<DT>::k32(a.w32[s], b.w32[s], acc);
    if (RowOperand<C>::k16) acc = Mma<DT>::k16(a.w16[0], b.w16[0], acc);
    return acc;
}

__device__ inline float xor_max(float x) {
    x = fmaxf(x, __shfl_xor(x, 16));
    return fmaxf(x, __shfl_xor(x, 32));
}
__device__ inline float xor_sum(float x) {
    x += __shfl_xor(x, 16);
    return x + __shfl_xor(x, 32);
}

// Work split: `strips` strips of `nt` tiles per sequence.
struct Split {
    int tiles, nt, strips;
    int64_t items;
};
inline Split make_split(int64_t B, int64_t T, int min_nt) {
    Split s;
    s.tiles = (int)((T + 15) / 16);
    const int64_t want_waves = 256 * 4 * 6;   // ~6 waves per SIMD over the whole chip
    int64_t strips = (want_waves + B - 1) / B;
    const int max_strips = (s.tiles + min_nt - 1) / min_nt;
    if (strips > max_strips) strips = max_strips;
    if (strips < 1) strips = 1;
    s.nt = (int)((s.tiles + strips - 1) / strips);
    s.strips = (s.tiles + s.nt - 1) / s.nt;
    s.items = B * s.strips;
    return s;
}

// =============================================================================
// Fused forward
// =============================================================================
template <class DT, int C>
__global__ void __launch_bounds__(64 * kWaves)
fused_fwd_kernel(char *__restrict__ out, float *__restrict__ lse, const char *__restrict__ q,
                 const char *__restrict__ k, const char *__restrict__ v, const float *__restrict__ rpb,
                 const int32_t *__restrict__ t_valid, int64_t items, int T, int W, int L, int H, int tiles, int nt,
                 int strips, float scale) {
    using B = Blk<C>;
    constexpr int CT = C / 16;   // channel tiles of the output
    __shared__ __attribute__((aligned(16))) char smem[kWaves * 2 * kRing * B::kBytes];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t item = (int64_t)blockIdx.x * kWaves + wave;
    if (item >= items) return;
    const int64_t b = item / strips;
    const int strip = (int)(item - b * strips);
    const int i0 = strip * nt, i1 = min(i0 + nt, tiles);
    const int g = lane >> 4, n = lane & 15;

    LDS_PTR(char) kring = (LDS_PTR(char))smem + wave * (2 * kRing * B::kBytes);
    LDS_PTR(char) vring = kring + kRing * B::kBytes;
    const int64_t seq_off = b * (int64_t)T * (2 * C);
    const char *qs = q + seq_off, *ks = k + seq_off, *vs = v + seq_off;

    int tv = T;
    if (t_valid) tv = max(0, min(T, t_valid[b / H]));

    // log2-domain bias for the 12 slots of this lane: key - query = 16*(blk-1) + 4g + r - n
    const float *rpb_h = rpb ? rpb + (b % H) * W : nullptr;
    float bias[3][4];
#pragma unroll
    for (int blk = 0; blk < 3; ++blk)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int j = 16 * (blk - 1) + 4 * g + r - n + L;
            bias[blk][r] = (j >= 0 && j < W) ? (rpb_h ? rpb_h[j] * kLog2e : 0.f) : kNegInf;
        }
    const float scale2 = scale * kLog2e;

    // prologue: blocks i0-1, i0, i0+1 into the ring; Q of the first tile
    BlockRegs<C> kn, vn;
#pragma unroll
    for (int d = -1; d <= 1; ++d) {
        load_block<C>(kn, ks, i0 + d, T, lane);
        load_block<C>(vn, vs, i0 + d, T, lane);
        store_block<C>(kn, kring + ((i0 + d) & (kRing - 1)) * B::kBytes, lane);
        store_block<C>(vn, vring + ((i0 + d) & (kRing - 1)) * B::kBytes, lane);
    }
    RowOperand<C> qn;
    load_rows<C>(qn, qs, i0, T, lane);

    for (int i = i0; i < i1; ++i) {
        const RowOperand<C> qt = qn;
        // prefetch: block i+2 and the next Q tile
        const bool more = i + 1 < i1;
        if (more) {
            load_block<C>(kn, ks, i + 2, T, lane);
            load_block<C>(vn, vs, i + 2, T, lane);
            load_rows<C>(qn, qs, i + 1, T, lane);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // S^T for the three key blocks
        float z[3][4];
#pragma unroll
        for (int blk = 0; blk < 3; ++blk) {
            RowOperand<C> kop;
            read_rows<C>(kop, kring + ((i - 1 + blk) & (kRing - 1)) * B::kBytes, lane);
            const f32x4 s = dot_rows_mma<DT, C>(kop, qt);
#pragma unroll
            for (int r = 0; r < 4; ++r) z[blk][r] = __builtin_fmaf(s[r], scale2, bias[blk][r]);
        }

        // additive -100 of the model's mask, only on tiles that touch an edge
        const int qrow = 16 * i + n;
        float lse_shift = 0.f;
        if (16 * (i - 1) < 0 || 16 * (i + 2) > tv) {
            if (qrow >= tv) {
                lse_shift = kMaskValue;          // whole row shifted: softmax unchanged
            } else {
#pragma unroll
                for (int blk = 0; blk < 3; ++blk)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = 16 * (i - 1 + blk) + 4 * g + r;
                        if (key < 0 || key >= tv) z[blk][r] += kMaskValue * kLog2e;
                    }
            }
        }

        float m = z[0][0];
#pragma unroll
        for (int blk = 0; blk < 3; ++blk)
#pragma unroll
            for (int r = 0; r < 4; ++r) m = fmaxf(m, z[blk][r]);
        m = xor_max(m);

        float sum = 0.f;
        u32x2 pb[3];
#pragma unroll
        for (int blk = 0; blk < 3; ++blk) {
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                p[r] = __builtin_amdgcn_exp2f(z[blk][r] - m);
                sum += p[r];
            }
            pb[blk].x = Mma<DT>::pack(p[0], p[1]);
            pb[blk].y = Mma<DT>::pack(p[2], p[3]);
        }
        sum = xor_sum(sum);
        const float inv = __builtin_amdgcn_rcpf(sum);

        // O^T = sum over blocks of V_blk^T . P^T
        f32x4 o[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int blk = 0; blk < 3; ++blk) {
            LDS_PTR(char) slot = vring + ((i - 1 + blk) & (kRing - 1)) * B::kBytes;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) o[ct] = Mma<DT>::k16(read_tr<C>(slot, ct, lane), pb[blk], o[ct]);
        }

        if (qrow < T) {
            char *orow = out + seq_off + (int64_t)qrow * (2 * C);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                u32x2 w;
                w.x = Mma<DT>::pack(o[ct][0] * inv, o[ct][1] * inv);
                w.y = Mma<DT>::pack(o[ct][2] * inv, o[ct][3] * inv);
                *reinterpret_cast<u32x2 *>(orow + ct * 32 + g * 8) = w;
            }
            if (lse && g == 0) lse[b * (int64_t)T + qrow] = (m + __builtin_amdgcn_logf(sum)) * kLn2 + lse_shift;
        }

        // block i+2 replaces block i-2 in the ring
        if (more) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            store_block<C>(kn, kring + ((i + 2) & (kRing - 1)) * B::kBytes, lane);
            store_block<C>(vn, vring + ((i + 2) & (kRing - 1)) * B::kBytes, lane);
        }
    }
}

template <class DT, int C>
int launch_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
               const int32_t *t_valid, const Geom &g, float scale, hipStream_t s) {
    const Split sp = make_split(g.B, g.T, 4);
    const int64_t blocks = (sp.items + kWaves - 1) / kWaves;
    if (blocks > 0x7fffffffLL) return NA1D_ERR_SHAPE;
    fused_fwd_kernel<DT, C><<<(unsigned)blocks, 64 * kWaves, 0, s>>>(
        (char *)out, lse, (const char *)q, (const char *)k, (const char *)v, rpb, t_valid, sp.items, (int)g.T, g.W,
        g.L, g.H, sp.tiles, sp.nt, sp.strips, scale);
    return launch_status();
}

// Shapes the three-block kernels cover.
inline bool covered(const Geom &g) {
    const int R = g.W - 1 - g.L;
    if (g.L > 16 || R > 16) return false;
    if (g.C != 16 && g.C != 32 && g.C != 64 && g.C != 128) return false;
    if (g.T > (1 << 30) / g.C) return false;   // per-sequence byte offsets stay in 32 bits
    return true;
}

#define NA1D_MFMA_DISPATCH(FN, ...)                                            \
    do {                                                                       \
        if (dtype == NA1D_BF16) {                                              \
            switch (g.C) {                                                     \
                case 16: return FN<BF16, 16>(__VA_ARGS__);                     \
                case 32: return FN<BF16, 32>(__VA_ARGS__);                     \
                case 64: return FN<BF16, 64>(__VA_ARGS__);                     \
                case 128: return FN<BF16, 128>(__VA_ARGS__);                   \
            }                                                                  \
        } else {                                                               \
            switch (g.C) {                                                     \
                case 16: return FN<FP16, 16>(__VA_ARGS__);                     \
                case 32: return FN<FP16, 32>(__VA_ARGS__);                     \
                case 64: return FN<FP16, 64>(__VA_ARGS__);                     \
                case 128: return FN<FP16, 128>(__VA_ARGS__);                   \
            }                                                                  \
        }                                                                      \
        return NA1D_ERR_UNSUPPORTED;                                           \
    } while (0)

int fused_fwd(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
              const int32_t *t_valid, const Geom &g, float scale, int dtype, hipStream_t s) {
    if (!covered(g)) return NA1D_ERR_UNSUPPORTED;
    NA1D_MFMA_DISPATCH(launch_fwd, out, lse, q, k, v, rpb, t_valid, g, scale, s);
}

int qk(float *, const void *, const void *, const Geom &, int, hipStream_t) { return NA1D_ERR_UNSUPPORTED; }
int av(void *, const float *, const void *, const Geom &, int, hipStream_t) { return NA1D_ERR_UNSUPPORTED; }
int gather(void *, const float *, const void *, const Geom &, int, hipStream_t) { return NA1D_ERR_UNSUPPORTED; }
int fused_bwd(void *, void *, void *, float *, const void *, const void *, const void *, const void *, const void *,
              const float *, const float *, const int32_t *, const Geom &, float, int, hipStream_t) {
    return NA1D_ERR_UNSUPPORTED;
}

}  // namespace mfma
}  // namespace na1d
