// Stand-alone check of libna1d's C ABI: no Python, no torch, only the HIP runtime and include/na1d.h - the way a
// host program in any language binds the library.  Small seeded problems go through the six un-fused entry points,
// the fused forward and the dense forward, and are compared with index loops written out here in double precision
// (a restatement of the operator's definition that shares nothing with the library or with the Python oracle).
// Exit status 0 = every check passed.
//
// A second mode, `na1d_abi_check copy R W BYTES ITERS`, times a plain streaming copy: each launch reads R tensors
// of BYTES bytes, combines them and writes W tensors of BYTES bytes, with every buffer rotated over more than the
// last-level cache.  It is the yardstick a benchmark holds the operator's kernels against: what the memory system
// gives a kernel of this launch size that does nothing but move the same number of bytes.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <vector>

#include "na1d.h"

namespace {

#define HIP_OK(call)                                                              \
    do {                                                                          \
        if ((call) != hipSuccess) {                                               \
            std::printf("%s failed\n", #call);                                    \
            std::exit(3);                                                         \
        }                                                                         \
    } while (0)

uint16_t to_bf16(float x) {            // round to nearest even
    uint32_t u;
    std::memcpy(&u, &x, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float from_bf16(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float x;
    std::memcpy(&x, &u, 4);
    return x;
}

struct Rng {                           // xorshift64*, values in [-1, 1)
    uint64_t s;
    float next() {
        s ^= s >> 12;
        s ^= s << 25;
        s ^= s >> 27;
        return (float)((s * 0x2545F4914F6CDD1Dull) >> 40) / 8388608.0f - 1.0f;
    }
};

template <class T> T *to_device(const std::vector<T> &h) {
    T *d = nullptr;
    HIP_OK(hipMalloc(&d, h.size() * sizeof(T)));
    HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}
template <class T> std::vector<T> to_host(const T *d, size_t n) {
    std::vector<T> h(n);
    HIP_OK(hipMemcpy(h.data(), d, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
}

double rel_l2(const std::vector<double> &got, const std::vector<double> &want) {
    double num = 0, den = 0;
    for (size_t i = 0; i < got.size(); ++i) {
        num += (got[i] - want[i]) * (got[i] - want[i]);
        den += want[i] * want[i];
    }
    return std::sqrt(num / (den > 0 ? den : 1));
}

int failures = 0;
void expect(bool ok, const char *what, double value) {
    std::printf("%-34s %s (%.3g)\n", what, ok ? "ok" : "FAILED", value);
    if (!ok) ++failures;
}

std::vector<double> widen(const std::vector<uint16_t> &h) {
    std::vector<double> out(h.size());
    for (size_t i = 0; i < h.size(); ++i) out[i] = from_bf16(h[i]);
    return out;
}
std::vector<double> widen(const std::vector<float> &h) { return std::vector<double>(h.begin(), h.end()); }

int run(int N, int H, int T, int C, int W, int L) {
    const int B = N * H;
    const size_t rows = (size_t)B * T;
    Rng rng{0x9E3779B97F4A7C15ull ^ (uint64_t)(T * 131 + C * 7 + W)};
    std::vector<uint16_t> q(rows * C), k(rows * C), v(rows * C);
    for (auto *t : {&q, &k, &v})
        for (auto &x : *t) x = to_bf16(rng.next());
    std::vector<float> rpb((size_t)H * W), scores(rows * W);
    for (auto &x : rpb) x = 0.5f * rng.next();
    for (auto &x : scores) x = rng.next();
    std::vector<int32_t> t_valid(N);
    for (int n = 0; n < N; ++n) t_valid[n] = T - (n * T) / (2 * N);        // sample 0 unpadded, the others shorter
    const float scale = 1.0f / std::sqrt((float)C);
    auto at = [&](const std::vector<uint16_t> &x, int b, int t, int c) -> double {
        return (t < 0 || t >= T) ? 0.0 : (double)from_bf16(x[((size_t)b * T + t) * C + c]);      // zero fill
    };

    // ---- definitions, written out
    std::vector<double> p1(rows * W), p2(rows * C), p3(rows * C, 0.0), fused(rows * C), lse(rows), dense(rows * C);
    for (int b = 0; b < B; ++b)
        for (int t = 0; t < T; ++t) {
            std::vector<double> z(W), zd(T);
            const int tv = t_valid[b / H];
            for (int j = 0; j < W; ++j) {
                double s = 0;
                for (int c = 0; c < C; ++c) s += at(q, b, t, c) * at(k, b, t - L + j, c);
                p1[((size_t)b * T + t) * W + j] = s;
                const int u = t - L + j;
                z[j] = s * scale + rpb[(size_t)(b % H) * W + j] + ((t >= tv || u < 0 || u >= tv) ? -100.0 : 0.0);
            }
            double m = z[0];
            for (double x : z) m = std::fmax(m, x);
            double den = 0;
            for (double x : z) den += std::exp(x - m);
            lse[(size_t)b * T + t] = m + std::log(den);
            for (int c = 0; c < C; ++c) {
                double o = 0, a = 0;
                for (int j = 0; j < W; ++j) {
                    o += std::exp(z[j] - m) / den * at(v, b, t - L + j, c);
                    a += (double)scores[((size_t)b * T + t) * W + j] * at(v, b, t - L + j, c);
                }
                fused[((size_t)b * T + t) * C + c] = o;
                p2[((size_t)b * T + t) * C + c] = a;
            }
            for (int j = 0; j < W; ++j) {               // inverse-neighbourhood gather, as a scatter
                const int u = t - L + j;
                if (u < 0 || u >= T) continue;
                for (int c = 0; c < C; ++c)
                    p3[((size_t)b * T + u) * C + c] += (double)scores[((size_t)b * T + t) * W + j] * at(q, b, t, c);
            }
            double md = -1e300;
            for (int u = 0; u < T; ++u) {
                double s = 0;
                for (int c = 0; c < C; ++c) s += at(q, b, t, c) * at(k, b, u, c);
                zd[u] = s * scale + ((t >= tv || u >= tv) ? -100.0 : 0.0);
                md = std::fmax(md, zd[u]);
            }
            double dd = 0;
            for (int u = 0; u < T; ++u) dd += std::exp(zd[u] - md);
            for (int c = 0; c < C; ++c) {
                double o = 0;
                for (int u = 0; u < T; ++u) o += std::exp(zd[u] - md) / dd * at(v, b, u, c);
                dense[((size_t)b * T + t) * C + c] = o;
            }
        }

    // ---- the library
    uint16_t *dq = to_device(q), *dk = to_device(k), *dv = to_device(v);
    float *drpb = to_device(rpb), *dscores = to_device(scores);
    int32_t *dtv = to_device(t_valid);
    float *dattn = nullptr, *dlse = nullptr;
    uint16_t *dout = nullptr;
    HIP_OK(hipMalloc(&dattn, rows * W * 4));
    HIP_OK(hipMalloc(&dlse, rows * 4));
    HIP_OK(hipMalloc(&dout, rows * C * 2));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    std::printf("N=%d H=%d T=%d C=%d W=%d L=%d\n", N, H, T, C, W, L);
    auto status = [&](int st, const char *name) {
        if (st != NA1D_OK) std::printf("%s: %s\n", name, na1d_status_string(st));
        expect(st == NA1D_OK, name, st);
    };
    auto result16 = [&] { HIP_OK(hipStreamSynchronize(stream)); return widen(to_host(dout, rows * C)); };

    status(na1d_qk_forward(dattn, dq, dk, B, T, C, W, L, NA1D_BF16, stream), "na1d_qk_forward");
    HIP_OK(hipStreamSynchronize(stream));
    const double e1 = rel_l2(widen(to_host(dattn, rows * W)), p1);
    expect(e1 < 1e-5, "  band QK^T vs definition", e1);
    status(na1d_a_backward(dattn, dq, dk, B, T, C, W, L, NA1D_BF16, stream), "na1d_a_backward (alias of P1)");
    HIP_OK(hipStreamSynchronize(stream));
    expect(rel_l2(widen(to_host(dattn, rows * W)), p1) == e1, "  same bits as na1d_qk_forward", 0);

    status(na1d_av_forward(dout, dscores, dv, B, T, C, W, L, NA1D_BF16, stream), "na1d_av_forward");
    const double e2 = rel_l2(result16(), p2);
    expect(e2 < 1e-2, "  band . V vs definition", e2);
    status(na1d_q_backward(dout, dscores, dv, B, T, C, W, L, NA1D_BF16, stream), "na1d_q_backward (alias of P2)");
    expect(rel_l2(result16(), p2) == e2, "  same bits as na1d_av_forward", 0);

    status(na1d_k_backward(dout, dscores, dq, B, T, C, W, L, NA1D_BF16, stream), "na1d_k_backward");
    const double e3 = rel_l2(result16(), p3);
    expect(e3 < 1e-2, "  inverse gather vs definition", e3);
    status(na1d_v_backward(dout, dscores, dq, B, T, C, W, L, NA1D_BF16, stream), "na1d_v_backward (alias of P3)");
    expect(rel_l2(result16(), p3) == e3, "  same bits as na1d_k_backward", 0);

    status(na1d_fused_forward(dout, dlse, dq, dk, dv, drpb, dtv, B, H, T, C, W, L, scale, NA1D_BF16, stream),
           "na1d_fused_forward");
    const double e4 = rel_l2(result16(), fused);
    expect(e4 < 1e-2, "  fused forward vs definition", e4);
    const double e5 = rel_l2(widen(to_host(dlse, rows)), lse);
    expect(e5 < 1e-4, "  log-sum-exp vs definition", e5);

    const int st = na1d_global_forward(dout, nullptr, dq, dk, dv, dtv, B, H, T, C, scale, NA1D_BF16, 0.0f, 0, stream);
    status(st, "na1d_global_forward");
    const double e6 = rel_l2(result16(), dense);
    expect(e6 < 1e-2, "  dense attention vs definition", e6);

    expect(na1d_fused_forward(dout, dlse, dq, dk, nullptr, drpb, dtv, B, H, T, C, W, L, scale, NA1D_BF16, stream) ==
               NA1D_ERR_NULL, "null pointer is a status, not a fault", NA1D_ERR_NULL);
    for (void *p : {(void *)dq, (void *)dk, (void *)dv, (void *)drpb, (void *)dscores, (void *)dtv, (void *)dattn,
                    (void *)dlse, (void *)dout})
        HIP_OK(hipFree(p));
    HIP_OK(hipStreamDestroy(stream));
    return 0;
}

}  // namespace

namespace {

// ---- streaming-copy yardstick -------------------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kCopyThreads = 256;
// EPT 16-byte elements per thread and tensor: 4 KB, 8 KB or 16 KB per workgroup and tensor.  Which is fastest depends
// on the launch size (small launches want many small workgroups), so the yardstick is the best of the three.
// NTL: the loads carry the non-temporal (read-once) policy; without it they are plain loads, the policy the operator's
// strip copies have to use for rows that a neighbouring strip reads too.
template <int NR, int NW, int EPT, bool NTL>
__global__ void __launch_bounds__(kCopyThreads) copy_kernel(u32x4 *const *__restrict__ bufs, size_t n) {
    const size_t base = (size_t)blockIdx.x * EPT * kCopyThreads + threadIdx.x;
    u32x4 acc[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) acc[e] = u32x4{0, 0, 0, 0};
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const size_t i = base + (size_t)e * kCopyThreads;
            if (i < n) acc[e] ^= NTL ? __builtin_nontemporal_load(&bufs[r][i]) : bufs[r][i];
        }
#pragma unroll
    for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const size_t i = base + (size_t)e * kCopyThreads;
            acc[e].x += (uint32_t)w;
            if (i < n) __builtin_nontemporal_store(acc[e], &bufs[NR + w][i]);
        }
}

// Average kernel time in us of `iters` launches, every launch between its own pair of events recorded by the launch
// itself (the dispatch's begin and end), buffers rotated over `sets` sets.
template <int NR, int NW, int EPT, bool NTL> double time_copy_variant(const std::vector<u32x4 **> &dsets, size_t n, int iters) {
    const int sets = (int)dsets.size();
    const unsigned grid = (unsigned)((n + kCopyThreads * EPT - 1) / (kCopyThreads * EPT));
    for (int it = 0; it < sets + 3; ++it) copy_kernel<NR, NW, EPT, NTL><<<grid, kCopyThreads>>>(dsets[it % sets], n);
    HIP_OK(hipDeviceSynchronize());
    std::vector<hipEvent_t> ev(2 * (size_t)iters);
    for (auto &e : ev) HIP_OK(hipEventCreate(&e));
    for (int it = 0; it < iters; ++it)
        hipExtLaunchKernelGGL((copy_kernel<NR, NW, EPT, NTL>), dim3(grid), dim3(kCopyThreads), 0, nullptr, ev[2 * it],
                              ev[2 * it + 1], 0, dsets[it % sets], n);
    HIP_OK(hipDeviceSynchronize());
    double total = 0;
    for (int it = 0; it < iters; ++it) {
        float ms = 0;
        HIP_OK(hipEventElapsedTime(&ms, ev[2 * it], ev[2 * it + 1]));
        total += ms;
    }
    for (auto &e : ev) HIP_OK(hipEventDestroy(e));
    return total * 1e3 / iters;
}

template <int NR, int NW, bool NTL> int time_copy(size_t bytes, int iters) {
    const size_t n = bytes / 16;
    const int nb = NR + NW, sets = (int)std::min(64.0, 700e6 / ((double)nb * (double)bytes) + 2);
    std::vector<u32x4 **> dsets;
    for (int s = 0; s < sets; ++s) {
        std::vector<u32x4 *> h(nb);
        for (auto &p : h) {
            HIP_OK(hipMalloc(&p, bytes));
            HIP_OK(hipMemset(p, 1, bytes));
        }
        u32x4 **d = nullptr;
        HIP_OK(hipMalloc(&d, nb * sizeof(void *)));
        HIP_OK(hipMemcpy(d, h.data(), nb * sizeof(void *), hipMemcpyHostToDevice));
        dsets.push_back(d);
    }
    const double t1 = time_copy_variant<NR, NW, 1, NTL>(dsets, n, iters), t2 = time_copy_variant<NR, NW, 2, NTL>(dsets, n, iters),
                 t4 = time_copy_variant<NR, NW, 4, NTL>(dsets, n, iters);
    const double us = std::min(t1, std::min(t2, t4));
    std::printf("copy %dR+%dW x %zu bytes, %s loads, %d launches: copy_us=%.3f GBps=%.1f (per thread and tensor 1 / 2 / 4 x 16 B: "
                "%.3f / %.3f / %.3f us)\n", NR, NW, bytes, NTL ? "read-once" : "plain", iters, us,
                (double)nb * (double)bytes / us / 1e3, t1, t2, t4);
    return 0;
}

int copy_mode(int argc, char **argv) {
    if (argc != 6 && !(argc == 7 && std::strcmp(argv[6], "plain") == 0)) {
        std::printf("usage: %s copy READS WRITES BYTES ITERS [plain]   (plain: loads without the read-once policy)\n", argv[0]);
        return 64;
    }
    const bool plain = argc == 7;
    const int r = std::atoi(argv[2]), w = std::atoi(argv[3]), iters = std::atoi(argv[5]);
    const size_t bytes = (size_t)std::atoll(argv[4]) / 16 * 16;
    if (iters < 1 || iters > 10000 || bytes < 16 || bytes > ((size_t)1 << 31)) return 64;
    if (r == 3 && w == 1) return plain ? time_copy<3, 1, false>(bytes, iters) : time_copy<3, 1, true>(bytes, iters);
    if (r == 4 && w == 3) return plain ? time_copy<4, 3, false>(bytes, iters) : time_copy<4, 3, true>(bytes, iters);
    if (r == 2 && w == 1) return plain ? time_copy<2, 1, false>(bytes, iters) : time_copy<2, 1, true>(bytes, iters);
    if (r == 1 && w == 1) return plain ? time_copy<1, 1, false>(bytes, iters) : time_copy<1, 1, true>(bytes, iters);
    std::printf("copy: READS+WRITES must be 1+1, 2+1, 3+1 or 4+3\n");
    return 64;
}

}  // namespace

int main(int argc, char **argv) {
    if (argc > 1 && std::strcmp(argv[1], "copy") == 0) return copy_mode(argc, argv);
    std::printf("libna1d version %d\n", na1d_version());
    if (run(2, 2, 37, 16, 27, 13) || run(3, 1, 50, 32, 15, 7) || run(1, 2, 20, 64, 33, 16) || run(2, 1, 9, 24, 5, 0)) return 2;
    std::printf(failures ? "%d checks FAILED\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
