#!/usr/bin/env python3
"""NA1D benchmark on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is
already resident in HBM: the fused NA1D forward followed by the fused backward
(forward only for the forward-only workloads), called through the C ABI on
torch's current stream.  Inputs rotate over enough buffer sets to exceed the
256 MB Infinity Cache, so cache hits do not pose as HBM bandwidth.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2]

prints ONE JSON line.  `value` is algorithmic bytes per step / seconds per step
(GB/s): 8*C bytes per token forward, 14*C backward (q,k,v[,dO] read and
O / dQ,dK,dV written once, 16-bit; per-row statistics excluded).  Beside the
headline workload the line carries, under `configs`, the kernel time and the
fraction of the HBM roofline of the forward and backward kernels at every
configuration shape, in the packed [B,T,C] layout and in the head-interleaved
projection layout the models use, and under `unfused` the three kernels of the
reference's two-call API.

    python bench.py --only cfg3:strided --steps 200

runs nothing but that configuration's kernels (for a profiler) and prints its record.
"""
import argparse
import ctypes
import json
import os
import re
import statistics
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "pcf-nat_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0
ROTATE_BYTES = 600e6          # > 2x the 256 MB Infinity Cache in rotation
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "fused_kernels_hbm_traffic.md")

# name: (N, H, T, C, W, dtype, backward?)   [B = N*H]
WORKLOADS = {
    "cfg1": dict(N=32, H=4, T=200, C=64, W=7, dtype="bf16", bwd=False,
                 desc="NA1D fwd bf16 batch=32 heads=4 T=200 head_dim=64 window=7"),
    "cfg2": dict(N=128, H=8, T=300, C=32, W=15, dtype="fp16", bwd=True,
                 desc="NA1D fwd+bwd fp16 batch=128 heads=8 T=300 head_dim=32 window=15"),
    "cfg3": dict(N=256, H=16, T=100, C=16, W=27, dtype="bf16", bwd=False,
                 desc="NA layer of PCF-NAT 4x4 inference: batch=256 heads=16 T=100 head_dim=16 window=27, fwd bf16"),
    "cfg4": dict(N=64, H=16, T=1000, C=16, W=27, dtype="bf16", bwd=False,
                 desc="NA layer of PCF-NAT 6x4 at max length: batch=64 heads=16 T=1000 head_dim=16 window=27, fwd bf16"),
    "cfg5": dict(N=128, H=16, T=100, C=16, W=27, dtype="fp16", bwd=True,
                 desc="NA layer of MFA-NAT 4x4 training: batch=128 heads=16 T=100 head_dim=16 window=27, fwd+bwd fp16"),
}


def window_left(W):
    """Slots left of the query in an odd or even window: W - 1 - W // 2 (models/PCF_NATransformer.py:48-49)."""
    return W - 1 - W // 2


def algorithmic_bytes(w):
    tokens = w["N"] * w["H"] * w["T"]
    fwd = 8 * w["C"] * tokens
    bwd = 14 * w["C"] * tokens if w["bwd"] else 0
    return fwd, bwd


def short_kernel_name(name):
    """A kernel's name without return type, namespaces and argument list, spaces removed: the key under which
    the library, a kernel trace and the traffic table agree."""
    name = name.strip().strip('"')
    name = re.sub(r"^void\s+", "", name)
    name = re.sub(r"\(.*$", "", name)
    name = re.sub(r"\b(?:na1d|mfma)::", "", name)
    return name.replace(" ", "")


def measured_traffic(workload, kernel, path=TRAFFIC_FILE):
    """HBM bytes per launch of `kernel` at `workload` from the committed rocprofv3 --pmc summary: a markdown table
    whose rows read | workload | kernel | FETCH_SIZE KiB | factor | WRITE_SIZE KiB | factor | ...  Returns None when
    the file has no row for exactly this workload and kernel (a kernel that changed its name has not been measured)."""
    if not os.path.exists(path):
        return None
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) < 6 or cells[0] != workload:
            continue
        if short_kernel_name(cells[1].strip("`")) != short_kernel_name(kernel):
            continue
        try:
            fetch, ffac, write, wfac = (float(cells[i]) for i in (2, 3, 4, 5))
        except ValueError:
            continue
        return int((fetch * ffac + write * wfac) * 1024)
    return None


# ---------------------------------------------------------------------------------------------------------------
# buffers
# ---------------------------------------------------------------------------------------------------------------
def _dtype(w):
    import torch
    return torch.bfloat16 if w["dtype"] == "bf16" else torch.float16


def n_sets_for(w):
    fwd, bwd = algorithmic_bytes(w)
    return max(2, int(ROTATE_BYTES // (fwd + bwd)) + 1)


def make_packed_sets(w, n_sets, device):
    import torch
    dt = _dtype(w)
    B, T, C = w["N"] * w["H"], w["T"], w["C"]
    g = torch.Generator(device="cpu").manual_seed(0)
    sets = []
    for _ in range(n_sets):
        s = {}
        for name in ("q", "k", "v", "do"):
            s[name] = torch.randn(B, T, C, generator=g, dtype=torch.float32).to(dt).to(device)
        s["q"] = s["q"] * (C ** -0.5)
        s["rpb"] = (torch.randn(w["H"], w["W"], generator=g) * 0.02).to(device)
        s["o"] = torch.empty_like(s["q"])
        s["lse"] = torch.empty(B, T, dtype=torch.float32, device=device)
        if w["bwd"]:
            for name in ("dq", "dk", "dv"):
                s[name] = torch.empty_like(s["q"])
            s["drpb"] = torch.zeros(w["H"], w["W"], dtype=torch.float32, device=device)
        sets.append(s)
    return sets


def make_strided_sets(w, n_sets, device):
    """The layout the models hand over: qkv [N, T, 3, H, C] (the projection's output), out [N, T, H*C]."""
    import torch
    dt = _dtype(w)
    N, H, T, C = w["N"], w["H"], w["T"], w["C"]
    g = torch.Generator(device="cpu").manual_seed(0)
    sets = []
    for _ in range(n_sets):
        s = {"qkv": torch.randn(N, T, 3, H, C, generator=g, dtype=torch.float32).to(dt).to(device),
             "rpb": (torch.randn(H, w["W"], generator=g) * 0.02).to(device),
             "o": torch.empty(N, T, H * C, dtype=dt, device=device),
             "lse": torch.empty(N * H, T, dtype=torch.float32, device=device)}
        if w["bwd"]:
            s["do"] = torch.randn(N, T, H * C, generator=g, dtype=torch.float32).to(dt).to(device)
            s["dqkv"] = torch.empty_like(s["qkv"])
            s["drpb"] = torch.zeros(H, w["W"], dtype=torch.float32, device=device)
        sets.append(s)
    return sets


# ---------------------------------------------------------------------------------------------------------------
# kernel timing with the library's own events
# ---------------------------------------------------------------------------------------------------------------
class KernelClock:
    """Times single kernels with pairs of HIP events that the library records tightly around the kernel
    (na1d_profile_events -> hipExtLaunchKernel: the dispatch's begin and end on the launch stream, the interval a
    profiler's kernel trace reports, without the gaps between launches)."""

    def __init__(self, lib):
        self.lib = lib
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.pool = []

    def _pair(self, i):
        while len(self.pool) <= i:
            a, b = ctypes.c_void_p(), ctypes.c_void_p()
            assert self.hip.hipEventCreate(ctypes.byref(a)) == 0 and self.hip.hipEventCreate(ctypes.byref(b)) == 0
            self.pool.append((a, b))
        return self.pool[i]

    def _elapsed_ms(self, pair):
        ms = ctypes.c_float()
        assert self.hip.hipEventElapsedTime(ctypes.byref(ms), pair[0], pair[1]) == 0
        return ms.value

    def run(self, calls, steps):
        """calls: list of functions f(i) that each launch ONE kernel; they are called in turn for i in
        range(steps).  Returns per call (mean ms, name of the kernel it launched)."""
        import torch
        n = len(calls)
        for i in range(steps):
            for j, f in enumerate(calls):
                self.lib.na1d_profile_events(*self._pair(i * n + j))
                f(i)
        names = []
        for j, f in enumerate(calls):       # which kernel each call launches (one more launch each)
            self.lib.na1d_profile_events(*self._pair(steps * n + j))
            f(0)
            names.append(self.lib.na1d_profile_last_kernel().decode())
        self.lib.na1d_profile_events(None, None)
        torch.cuda.synchronize()
        return [(statistics.mean(self._elapsed_ms(self.pool[i * n + j]) for i in range(steps)), names[j])
                for j in range(n)]

    def close(self):
        for a, b in self.pool:
            self.hip.hipEventDestroy(a)
            self.hip.hipEventDestroy(b)
        self.pool = []


def bind_packed(lib, w, sets, with_lse=True):
    """Argument tuples bound once, so that a timed call is one ctypes call."""
    import torch
    from na1d_amd import _lib
    H, T, C, W = w["H"], w["T"], w["C"], w["W"]
    B = w["N"] * H
    L = window_left(W)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tag = _lib.dtype_tag(sets[0]["q"].dtype)
    n = len(sets)
    fa = [(P(s["o"]), P(s["lse"]) if with_lse else None, P(s["q"]), P(s["k"]), P(s["v"]), P(s["rpb"]), None, B, H, T, C,
           W, L, 1.0, tag, stream) for s in sets]
    fwd = lambda i: _lib.check(lib.na1d_fused_forward(*fa[i % n]), "na1d_fused_forward")
    bwd = None
    if w["bwd"]:
        ba = [(P(s["dq"]), P(s["dk"]), P(s["dv"]), P(s["drpb"]), P(s["q"]), P(s["k"]), P(s["v"]), P(s["o"]), P(s["do"]),
               P(s["lse"]), P(s["rpb"]), None, B, H, T, C, W, L, 1.0, tag, None, 0, stream) for s in sets]
        bwd = lambda i: _lib.check(lib.na1d_fused_backward(*ba[i % n]), "na1d_fused_backward")
    return fwd, bwd


def bind_strided(lib, w, sets, with_lse=True, which="both"):
    """`which`: "both" = projection layout in and out; "in" / "out" = only that side head-interleaved, the other
    packed (the same bytes; separates what the reads cost from what the writes cost)."""
    import torch
    from na1d_amd import _lib
    N, H, T, C, W = w["N"], w["H"], w["T"], w["C"], w["W"]
    L = window_left(W)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tag = _lib.dtype_tag(sets[0]["qkv"].dtype)
    i64x3 = ctypes.c_int64 * 3
    qs, os_ = i64x3(T * 3 * H * C, C, 3 * H * C), i64x3(T * H * C, C, H * C)
    step = H * C * 2
    if which == "out":      # q, k, v packed [N*H, T, C] one behind the other in the same buffer
        qs, step = i64x3(H * T * C, T * C, C), N * H * T * C * 2
    if which == "in":
        os_ = i64x3(H * T * C, T * C, C)
    n = len(sets)

    def parts(t):
        base = t.data_ptr()
        return ctypes.c_void_p(base), ctypes.c_void_p(base + step), ctypes.c_void_p(base + 2 * step)

    fa = [(P(s["o"]), P(s["lse"]) if with_lse else None, *parts(s["qkv"]), P(s["rpb"]), None, N, H, T, C, W, L, 1.0, tag,
           qs, os_, stream) for s in sets]
    fwd = lambda i: _lib.check(lib.na1d_fused_forward_strided(*fa[i % n]), "na1d_fused_forward_strided")
    bwd = None
    if w["bwd"]:
        ba = [(*parts(s["dqkv"]), P(s["drpb"]), *parts(s["qkv"]), P(s["do"]), P(s["lse"]), P(s["rpb"]), None, N, H, T, C,
               W, L, 1.0, tag, qs, os_, None, 0, stream) for s in sets]
        bwd = lambda i: _lib.check(lib.na1d_fused_backward_strided(*ba[i % n]), "na1d_fused_backward_strided")
    return fwd, bwd


def kernel_record(ms, name, nbytes, workload=None):
    gbps = nbytes / (ms * 1e-3) / 1e9
    rec = {"kernel": name, "kernel_us": round(ms * 1e3, 3), "algorithmic_bytes": nbytes, "GBps": round(gbps, 1),
           "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4)}
    if workload:
        rec["hbm_traffic_bytes"] = measured_traffic(workload, name)
    return rec


def config_record(lib, clock, name, layout, steps, warmup, device):
    """Forward (and backward) kernel time of one configuration shape in one layout."""
    import torch
    w = WORKLOADS[name]
    n_sets = n_sets_for(w)
    if layout == "packed":
        fwd, bwd = bind_packed(lib, w, make_packed_sets(w, n_sets, device), with_lse=w["bwd"])
    else:
        which = {"strided": "both", "strided_in": "in", "strided_out": "out"}[layout]
        fwd, bwd = bind_strided(lib, w, make_strided_sets(w, n_sets, device), with_lse=w["bwd"], which=which)
    calls = [fwd] + ([bwd] if bwd else [])
    for i in range(max(warmup, n_sets)):
        for f in calls:
            f(i)
    torch.cuda.synchronize()
    timed = clock.run(calls, steps)
    fb, bb = algorithmic_bytes(w)
    label = name if layout == "packed" else name + ":" + layout      # the traffic table's workload column
    rec = {"name": name, "layout": layout, "B": w["N"] * w["H"], "T": w["T"], "C": w["C"], "W": w["W"],
           "dtype": w["dtype"], "launches": steps, "forward": kernel_record(*timed[0], fb, label),
           "backward": kernel_record(*timed[1], bb, label) if bwd else None}
    torch.cuda.empty_cache()
    return rec


def unfused_record(lib, clock, name, steps, warmup, device):
    """The three kernels behind the reference's two-call API (QK / AV / inverse gather) at one configuration shape:
    4C + 4W algorithmic bytes per token each (16-bit rows in or out, fp32 scores out or in)."""
    import torch
    from na1d_amd import _lib
    w = WORKLOADS[name]
    H, T, C, W = w["H"], w["T"], w["C"], w["W"]
    B = w["N"] * H
    L = window_left(W)
    dt = _dtype(w)
    nbytes = B * T * (4 * C + 4 * W)
    n = max(2, int(ROTATE_BYTES // nbytes) + 1)
    g = torch.Generator(device="cpu").manual_seed(0)
    rows = [torch.randn(B, T, C, generator=g).to(dt).to(device) for _ in range(n)]
    other = [torch.randn(B, T, C, generator=g).to(dt).to(device) for _ in range(n)]
    outs = [torch.empty(B, T, C, dtype=dt, device=device) for _ in range(n)]
    attn = [torch.softmax(torch.randn(B, T, W, generator=g), -1).to(device) for _ in range(n)]
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tag = _lib.dtype_tag(dt)
    tail = (B, T, C, W, L, tag, stream)
    qk = lambda i: _lib.check(lib.na1d_qk_forward(P(attn[i % n]), P(rows[i % n]), P(other[i % n]), *tail), "qk")
    av = lambda i: _lib.check(lib.na1d_av_forward(P(outs[i % n]), P(attn[i % n]), P(rows[i % n]), *tail), "av")
    ga = lambda i: _lib.check(lib.na1d_k_backward(P(outs[i % n]), P(attn[i % n]), P(rows[i % n]), *tail), "gather")
    rec = {"name": name, "B": B, "T": T, "C": C, "W": W, "dtype": w["dtype"], "launches": steps}
    for key, f in (("qk_forward", qk), ("av_forward", av), ("k_backward", ga)):     # one at a time: each owns the cache
        for i in range(max(warmup, n)):
            f(i)
        torch.cuda.synchronize()
        (ms, kname), = clock.run([f], steps)
        rec[key] = kernel_record(ms, kname, nbytes)
    del rows, other, outs, attn
    torch.cuda.empty_cache()
    return rec


MFMA_PEAK_TFLOPS = 2500.0      # dense bf16 / fp16 matrix-core peak of MI355X

# Windows the two/three-block kernels do not cover run the wide kernels: the reference allows up to 80 slots
# (models/PCF_NATransformer.py:53).  name: (N, H, T, C, W, dtype)
WIDE_WORKLOADS = {
    "wide33": dict(N=128, H=8, T=300, C=32, W=33, dtype="fp16", bwd=True,
                   desc="NA1D fwd+bwd fp16 batch=128 heads=8 T=300 head_dim=32 window=33 (wide-window kernels)"),
    "wide65": dict(N=128, H=8, T=300, C=32, W=65, dtype="fp16", bwd=True,
                   desc="NA1D fwd+bwd fp16 batch=128 heads=8 T=300 head_dim=32 window=65 (wide-window kernels)"),
}

# The two dense (GlobalAttention) layers of each model (models/PCF_NATransformer.py:181-225): 4 heads of 64 channels.
GLOBAL_WORKLOADS = {
    "global_cfg3": dict(N=256, H=4, T=100, C=64, dtype="bf16", bwd=False,
                        desc="dense layer of PCF-NAT 4x4 inference: batch=256 heads=4 T=100 head_dim=64, fwd bf16"),
    "global_cfg4": dict(N=64, H=4, T=1000, C=64, dtype="bf16", bwd=False,
                        desc="dense layer of PCF-NAT 6x4 at max length: batch=64 heads=4 T=1000 head_dim=64, fwd bf16"),
    "global_cfg5": dict(N=128, H=4, T=100, C=64, dtype="fp16", bwd=True,
                        desc="dense layer of MFA-NAT 4x4 training: batch=128 heads=4 T=100 head_dim=64, fwd+bwd fp16"),
}


def wide_record(lib, clock, name, steps, warmup, device):
    """Forward and backward kernel of one wide-window shape (packed layout), bytes as for the other fused kernels."""
    import torch
    w = WIDE_WORKLOADS[name]
    n_sets = n_sets_for(w)
    fwd, bwd = bind_packed(lib, w, make_packed_sets(w, n_sets, device), with_lse=True)
    for i in range(max(warmup, n_sets)):
        fwd(i)
        bwd(i)
    torch.cuda.synchronize()
    timed = clock.run([fwd, bwd], steps)
    fb, bb = algorithmic_bytes(w)
    rec = {"name": name, "workload": w["desc"], "B": w["N"] * w["H"], "T": w["T"], "C": w["C"], "W": w["W"],
           "dtype": w["dtype"], "launches": steps, "forward": kernel_record(*timed[0], fb),
           "backward": kernel_record(*timed[1], bb)}
    torch.cuda.empty_cache()
    return rec


def global_record(lib, clock, name, steps, warmup, device):
    """Dense attention at one of the models' shapes.  At a thousand rows a sequence the kernels are bound by the matrix
    and vector instructions, at a hundred they are short memory-bound launches: the record gives TFLOP/s against the
    dense 16-bit matrix-core peak, counting 4*T*T*C flop per sequence forward (Q.K^T and P.V) and 10*T*T*C backward
    (five products of that size), next to the bytes moved and their rate."""
    import torch
    from na1d_amd import _lib
    w = GLOBAL_WORKLOADS[name]
    N, H, T, C = w["N"], w["H"], w["T"], w["C"]
    B, dt = N * H, _dtype(w)
    n = max(2, int(ROTATE_BYTES // (B * T * C * 2 * (11 if w["bwd"] else 4))) + 1)
    g = torch.Generator(device="cpu").manual_seed(0)
    sets = []
    for _ in range(n):
        st = {k_: torch.randn(B, T, C, generator=g).to(dt).to(device) for k_ in ("q", "k", "v", "do")}
        st["o"], st["lse"] = torch.empty_like(st["q"]), torch.empty(B, T, dtype=torch.float32, device=device)
        if w["bwd"]:
            for k_ in ("dq", "dk", "dv"):
                st[k_] = torch.empty_like(st["q"])
            st["ws"] = torch.empty(_lib.global_backward_workspace_bytes(B, H, T, C, dt), dtype=torch.uint8, device=device)
        sets.append(st)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tag, scale = _lib.dtype_tag(dt), C ** -0.5
    fa = [(P(s["o"]), P(s["lse"]), P(s["q"]), P(s["k"]), P(s["v"]), None, B, H, T, C, scale, tag, 0.0, 0, stream) for s in sets]
    fwd = lambda i: _lib.check(lib.na1d_global_forward(*fa[i % n]), "na1d_global_forward")
    calls = [fwd]
    if w["bwd"]:
        ba = [(P(s["dq"]), P(s["dk"]), P(s["dv"]), P(s["q"]), P(s["k"]), P(s["v"]), P(s["o"]), P(s["do"]), P(s["lse"]), None,
               B, H, T, C, scale, tag, 0.0, 0, P(s["ws"]), s["ws"].numel(), stream) for s in sets]
        calls.append(lambda i: _lib.check(lib.na1d_global_backward(*ba[i % n]), "na1d_global_backward"))
    for i in range(max(warmup, n)):
        for f in calls:
            f(i)
    torch.cuda.synchronize()
    timed = clock.run(calls, steps)

    def rec_of(ms, kname, flop, nbytes):
        return {"kernel": kname, "kernel_us": round(ms * 1e3, 3), "flop": flop, "TFLOPs": round(flop / (ms * 1e-3) / 1e12, 2),
                "frac_of_mfma_peak": round(flop / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "algorithmic_bytes": nbytes,
                "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1)}

    rec = {"name": name, "workload": w["desc"], "B": B, "T": T, "C": C, "dtype": w["dtype"], "launches": steps,
           "forward": rec_of(*timed[0], 4 * T * T * C * B, 8 * C * B * T),
           "backward": rec_of(*timed[1], 10 * T * T * C * B, (18 * C + 8) * B * T) if w["bwd"] else None}
    del sets
    torch.cuda.empty_cache()
    return rec


def copy_yardstick(shapes, iters=100):
    """A plain streaming copy of the same byte volume (r reads + w writes of one tensor's bytes), timed by the
    stand-alone host program the library ships with (pcf-nat_amd/lib/na1d_abi_check copy ...): what the memory
    system gives a kernel that does nothing else, at this launch size.  Returns {label: record}."""
    exe = os.path.join(ROOT, "pcf-nat_amd", "lib", "na1d_abi_check")
    out = {}
    if not os.path.exists(exe):
        return {"error": "na1d_abi_check not built"}
    for label, (reads, writes, nbytes) in shapes.items():
        try:
            r = subprocess.run([exe, "copy", str(reads), str(writes), str(nbytes), str(iters)], capture_output=True,
                               text=True, timeout=120)
            m = re.search(r"copy_us=([0-9.]+)", r.stdout)
            if r.returncode != 0 or not m:
                out[label] = {"error": (r.stdout + r.stderr)[-200:]}
                continue
            us = float(m.group(1))
            total = (reads + writes) * nbytes
            out[label] = {"reads": reads, "writes": writes, "tensor_bytes": nbytes, "kernel_us": round(us, 3),
                          "GBps": round(total / us / 1e3, 1), "frac_of_hbm_peak": round(total / us / 1e3 / HBM_PEAK_GBPS, 4)}
            # the same copy with plain loads: the policy a kernel has to use for rows that another workgroup reads too
            r = subprocess.run([exe, "copy", str(reads), str(writes), str(nbytes), str(iters), "plain"],
                               capture_output=True, text=True, timeout=120)
            m = re.search(r"copy_us=([0-9.]+)", r.stdout)
            if r.returncode == 0 and m:
                out[label]["plain_loads_kernel_us"] = round(float(m.group(1)), 3)
        except Exception as e:
            out[label] = {"error": "%s: %s" % (type(e).__name__, str(e)[:200])}
    return out


# ---------------------------------------------------------------------------------------------------------------
# CPU baselines
# ---------------------------------------------------------------------------------------------------------------
def cpu_threads():
    """Threads for the CPU baselines: every core this process may use.  On a shared host that is the scheduler
    affinity / the OMP_NUM_THREADS the operator set, not os.cpu_count() (the whole machine)."""
    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    env = os.environ.get("OMP_NUM_THREADS", "")
    if env.isdigit() and int(env) > 0:
        avail = min(avail, int(env))
    return max(1, avail)


def cpu_baseline(w, budget_s=15.0):
    """The oracle (CPU restatement of the reference math, PyTorch fp32) timed on
    this host's cores on a bounded sample of the same workload."""
    import torch
    from oracle import na1d_oracle as O
    threads = cpu_threads()
    torch.set_num_threads(threads)
    H, T, C, W = w["H"], w["T"], w["C"], w["W"]
    _, L = O.split_window(W)
    n_sample = max(1, min(w["N"], 64))
    B = n_sample * H
    q, k, v, do = O.seeded_qkv(B, T, C, seed=0, dtype=torch.float32, n=4)
    rpb = torch.zeros(H, W)

    def run():
        if w["bwd"]:
            O.na1d_forward(q, k, v, W, L, rpb, None, H)
            O.na1d_backward_formulas(q, k, v, do, W, L, rpb, None, H)
        else:
            O.na1d_forward(q, k, v, W, L, rpb, None, H)

    run()
    times, t_start = [], time.perf_counter()
    while len(times) < 5 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    sec = statistics.median(times)
    fwd_b, bwd_b = algorithmic_bytes(dict(w, N=n_sample))
    return {"value": (fwd_b + bwd_b) / sec / 1e9, "unit": "GB/s", "cores": threads, "host_cpu_count": os.cpu_count(),
            "torch_threads": torch.get_num_threads(), "kind": "port",
            "sample": "%d of %d samples (B=%d rows of T=%d), median of %d runs after one warm-up, %.3f s each, "
                      "PyTorch CPU fp32 on the %d cores this process may use (the host has %d)"
                      % (n_sample, w["N"], B, T, len(times), sec, threads, os.cpu_count() or 0)}


def oracle_attention(q, k, v, W, L, rpb=None, t_valid=None, num_heads=1):
    """CPU attention for the baseline twin of the model (the product has no CPU path)."""
    import torch
    from oracle import na1d_oracle as O
    pad = None if t_valid is None else (q.shape[1] - t_valid).to(torch.int64)
    return O.na1d_forward(q, k, v, W, L, rpb.reshape(num_heads, W), pad, num_heads)[0]


def model_inference(batch=256, frames=200, steps=10, warmup=3, cpu=True, modes=("fused_qkv", "fused", "unfused"),
                    small_batches=True):
    """PCF-NAT 4x4 inference (the reference's configs/pcf_nat4x4.yaml, batch 256 x 200 frames): bf16 autocast,
    random-init weights, 80-dim fbank-shaped N(0,1) input with the mean over time removed.  Returns embeddings/s
    on the GPU for each way of running the 14 NA layers and, as a baseline, of the same model in PyTorch CPU fp32
    on a bounded batch."""
    import torch
    from na1d_amd import models
    torch.manual_seed(0)
    twin = models.PCF_NATransformer(na=oracle_attention, dtype=torch.bfloat16).eval()
    x = torch.randn(batch, 80, frames, generator=torch.Generator().manual_seed(1))
    x = x - x.mean(-1, keepdim=True)
    xd = x.cuda()
    rates, out, gpu = {}, None, None
    # "fused_qkv": the operator reads the qkv projection in place (no head split / merge copies) - the headline;
    # "fused": the reference's data flow (pack heads, scale q, fused operator, merge heads);
    # "unfused": the reference's own call sequence through the drop-in QK / AV functions (scores in memory).
    for na in modes:
        m = models.PCF_NATransformer(na=na, dtype=torch.bfloat16)
        m.load_state_dict(twin.state_dict())
        m = m.cuda().eval()
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
            for _ in range(warmup):
                y = m(xd)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                y = m(xd)
            torch.cuda.synchronize()
            rates[na] = (time.perf_counter() - t0) / steps
        if na == modes[0]:
            out, gpu = y, m
    sec = rates[modes[0]]
    res = {"model": "PCF-NAT 4x4", "batch": batch, "frames": frames, "dtype": "bf16", "steps": steps,
           "attention": modes[0], "ms_per_batch": round(sec * 1e3, 3), "embeddings_per_s": round(batch / sec, 1)}
    if "fused" in rates:
        res["embeddings_per_s_with_head_copies"] = round(batch / rates["fused"], 1)
    if "unfused" in rates:
        res["embeddings_per_s_unfused_dropin"] = round(batch / rates["unfused"], 1)
    if small_batches:
        # small batches are bound by launch overhead, not by the GPU: the same pass replayed from a captured HIP graph
        from na1d_amd.graphs import GraphedInference
        small = {}
        try:
            for nb in (1, 8):
                xs = xd[:nb].contiguous()
                graphed = GraphedInference(gpu, xs)

                def eager():
                    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                        return gpu(xs)
                for name, fn in (("eager_ms", eager), ("graph_ms", lambda: graphed(xs))):
                    for _ in range(3):
                        fn()
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    for _ in range(20):
                        fn()
                    torch.cuda.synchronize()
                    small.setdefault("batch_%d" % nb, {})[name] = round((time.perf_counter() - t0) / 20 * 1e3, 3)
        except Exception as e:      # an extra record: it must not take the headline line down with it
            small["error"] = "%s: %s" % (type(e).__name__, str(e)[:200])
        res["small_batch_latency"] = small
    if cpu:
        threads = cpu_threads()
        torch.set_num_threads(threads)
        nb = 16
        with torch.no_grad():
            ref = twin(x[:nb])                      # warm-up
            times = []
            for _ in range(5):
                t0 = time.perf_counter()
                ref = twin(x[:nb])
                times.append(time.perf_counter() - t0)
        csec = statistics.median(times)
        cos = torch.nn.functional.cosine_similarity(out[:nb].float().cpu(), ref, dim=-1).min().item()
        res["cpu_baseline"] = {"embeddings_per_s": round(nb / csec, 2), "cores": threads,
                               "host_cpu_count": os.cpu_count(), "kind": "port",
                               "sample": "batch %d of %d, median of 5 passes after one warm-up, PyTorch CPU fp32" % (nb, batch)}
        res["min_cosine_vs_cpu_twin"] = round(cos, 5)
    return res


# ---------------------------------------------------------------------------------------------------------------
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-model", action="store_true", help="skip the PCF-NAT 4x4 embeddings/s leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-configuration kernel records")
    ap.add_argument("--model-only", action="store_true",
                    help="run only batch-256 passes of PCF-NAT 4x4 with the in-place operator and print the record")
    ap.add_argument("--only", default=None, metavar="CFG[:LAYOUT]",
                    help="run only the kernels of one configuration (layout packed, strided or unfused) and print its record")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the op shards over "
              "batch*heads with no exchange between GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from na1d_amd import _lib

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    lib = _lib.load()
    dev = torch.device("cuda:0")
    if args.model_only:
        print(json.dumps(model_inference(steps=max(args.steps, 1) if args.steps != 200 else 10, cpu=False,
                                         modes=("fused_qkv",), small_batches=False)))
        return
    clock = KernelClock(lib)
    if args.only:
        name, _, layout = args.only.partition(":")
        layout = layout or "packed"
        if name in WIDE_WORKLOADS:
            print(json.dumps(wide_record(lib, clock, name, args.steps, args.warmup, dev)))
        elif name in GLOBAL_WORKLOADS:
            print(json.dumps(global_record(lib, clock, name, args.steps, args.warmup, dev)))
        elif layout == "unfused":
            print(json.dumps(unfused_record(lib, clock, name, args.steps, args.warmup, dev)))
        else:
            print(json.dumps(config_record(lib, clock, name, layout, args.steps, args.warmup, dev)))
        return

    w = WORKLOADS[args.workload]
    H, T, C, W = w["H"], w["T"], w["C"], w["W"]
    B = w["N"] * H
    L = window_left(W)
    fwd_bytes, bwd_bytes = algorithmic_bytes(w)
    set_bytes = fwd_bytes + bwd_bytes
    n_sets = n_sets_for(w)
    sets = make_packed_sets(w, n_sets, dev)
    fwd, bwd = bind_packed(lib, w, sets)

    for i in range(max(args.warmup, 1)):
        fwd(i)
        if bwd:
            bwd(i)
    torch.cuda.synchronize()

    # timed region: exactly K steps between two synchronisations, nothing else in the stream
    K = args.steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(K):
        fwd(i)
        if bwd:
            bwd(i)
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    ms_per_step = sec / K * 1e3

    # the same K steps again, every launch bracketed by its own pair of library events
    timed = clock.run([fwd] + ([bwd] if bwd else []), K)
    fwd_ms, fwd_name = timed[0]
    bwd_ms, bwd_name = timed[1] if bwd else (None, None)

    # for comparison: K back-to-back launches of the dominant kernel between two stream events (this average
    # includes the gap between consecutive launches)
    dom = bwd if bwd else fwd
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(K):
        dom(i)
    e1.record()
    torch.cuda.synchronize()
    back_to_back_ms = e0.elapsed_time(e1) / K
    dom_ms, dom_kernel = (bwd_ms, bwd_name) if bwd else (fwd_ms, fwd_name)

    value = set_bytes / (sec / K) / 1e9
    dom_name, dom_bytes = ("fused backward", bwd_bytes) if bwd else ("fused forward", fwd_bytes)
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    line = {
        "metric": "NA1D fwd+bwd HBM GB/s (% of peak); PCF-NAT 4x4 embeddings/sec on 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": w["desc"], "name": args.workload, "B": B, "T": T, "C": C, "W": W, "left": L,
                   "buffer_sets_rotated": n_sets, "algorithmic_bytes_per_step": set_bytes,
                   "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": measured_traffic(args.workload, dom_kernel),
                     "traffic_source": os.path.relpath(TRAFFIC_FILE, ROOT),
                     "kernel": dom_name, "kernel_name": dom_kernel, "kernel_ms": round(dom_ms, 5),
                     "algorithmic_bytes": dom_bytes},
        "kernels_ms_in_step": {"fused_forward": round(fwd_ms, 5),
                               "fused_backward": None if bwd_ms is None else round(bwd_ms, 5),
                               "dominant_back_to_back_incl_gaps": round(back_to_back_ms, 5)},
    }
    del sets, fwd, bwd, dom
    torch.cuda.empty_cache()
    if not args.no_configs:
        per_cfg = max(50, min(K, 100))          # launches per kernel and configuration
        recs, unf, wide, dense = [], [], [], []
        try:
            for name in sorted(WORKLOADS):
                for layout in ("packed", "strided"):
                    recs.append(config_record(lib, clock, name, layout, per_cfg, 10, dev))
            for name in ("cfg2", "cfg3"):
                unf.append(unfused_record(lib, clock, name, per_cfg, 10, dev))
            for name in sorted(WIDE_WORKLOADS):
                wide.append(wide_record(lib, clock, name, per_cfg, 10, dev))
            for name in sorted(GLOBAL_WORKLOADS):
                dense.append(global_record(lib, clock, name, per_cfg, 10, dev))
        except Exception as e:      # extra records must not take the headline line down with them
            recs.append({"error": "%s: %s" % (type(e).__name__, str(e)[:300])})
        line["configs"] = recs
        line["unfused"] = unf
        line["wide"] = wide
        line["global"] = dense
        shapes = {}
        for name, cw in sorted(WORKLOADS.items()):
            one = cw["N"] * cw["H"] * cw["T"] * cw["C"] * 2
            shapes[name + " forward"] = (3, 1, one)
            if cw["bwd"]:
                shapes[name + " backward"] = (4, 3, one)
        line["copy_yardstick"] = copy_yardstick(shapes, per_cfg)
    clock.close()
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(w)
    if not args.no_model:
        torch.cuda.empty_cache()
        try:
            line["pcf_nat_4x4_inference"] = model_inference(cpu=not args.no_cpu_baseline)
        except Exception as e:      # the operator's line above stands on its own
            line["pcf_nat_4x4_inference"] = {"error": "%s: %s" % (type(e).__name__, str(e)[:300])}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
