#!/usr/bin/env python3
"""NA1D benchmark on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is
already resident in HBM: the fused NA1D forward followed by the fused backward
(forward only for the forward-only workload), called through the C ABI on
torch's current stream.  Inputs rotate over enough buffer sets to exceed the
256 MB Infinity Cache, so cache hits do not pose as HBM bandwidth.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2]

prints ONE JSON line.  `value` is algorithmic bytes per step / seconds per step
(GB/s): 8*C bytes per token forward, 14*C backward (q,k,v[,dO] read and
O / dQ,dK,dV written once, 16-bit; per-row statistics excluded).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "pcf-nat_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0

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

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs
# (KiB per dispatch, each scaled by what the same counter reads for a plain copy kernel of known
# size: x2.0 for FETCH_SIZE, x1.0 for WRITE_SIZE on this machine); None where not measured.
MEASURED_TRAFFIC_BYTES = {
    "cfg2": int((39084.5 * 2.0 + 57865.2) * 1024),     # fused backward: 80.0 MB read + 59.3 MB written
    "cfg3": int((19241.4 * 2.0 + 14400.0) * 1024),     # fused forward: 39.4 MB read + 14.7 MB written
}


def algorithmic_bytes(w):
    tokens = w["N"] * w["H"] * w["T"]
    fwd = 8 * w["C"] * tokens
    bwd = 14 * w["C"] * tokens if w["bwd"] else 0
    return fwd, bwd


def make_sets(w, n_sets, device):
    import torch
    dt = torch.bfloat16 if w["dtype"] == "bf16" else torch.float16
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


def cpu_baseline(w, budget_s=15.0):
    """The oracle (CPU restatement of the reference math, PyTorch fp32) timed on
    this host's cores on a bounded sample of the same workload."""
    import torch
    from oracle import na1d_oracle as O
    cores = os.cpu_count() or 1
    threads = min(cores, 16)
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
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    sec = statistics.median(times)
    fwd_b, bwd_b = algorithmic_bytes(dict(w, N=n_sample))
    return {"value": (fwd_b + bwd_b) / sec / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "%d of %d samples (B=%d rows of T=%d), median of %d runs, %.3f s each, PyTorch CPU fp32"
                      % (n_sample, w["N"], B, T, len(times), sec)}


def oracle_attention(q, k, v, W, L, rpb=None, t_valid=None, num_heads=1):
    """CPU attention for the baseline twin of the model (the product has no CPU path)."""
    import torch
    from oracle import na1d_oracle as O
    pad = None if t_valid is None else (q.shape[1] - t_valid).to(torch.int64)
    return O.na1d_forward(q, k, v, W, L, rpb.reshape(num_heads, W), pad, num_heads)[0]


def model_inference(batch=256, frames=200, steps=10, warmup=3, cpu=True, modes=("fused", "fused_qkv")):
    """PCF-NAT 4x4 inference (the reference's configs/pcf_nat4x4.yaml, batch 256 x 200 frames): bf16 autocast, random-init weights, 80-dim fbank-shaped
    N(0,1) input with the mean over time removed, fused NA1D in all 14 NA layers.  Returns embeddings/s on the
    GPU and, as a baseline, of the same model in PyTorch CPU fp32 on a bounded batch."""
    import torch
    from na1d_amd import models
    torch.manual_seed(0)
    twin = models.PCF_NATransformer(na=oracle_attention, dtype=torch.bfloat16).eval()
    x = torch.randn(batch, 80, frames, generator=torch.Generator().manual_seed(1))
    x = x - x.mean(-1, keepdim=True)
    xd = x.cuda()
    rates = {}
    # "fused_qkv": the operator reads the qkv projection in place (no head split / merge copies);
    # "fused": the reference's data flow (pack heads, scale q, operator, merge heads).  The first is reported.
    for na in modes:
        gpu = models.PCF_NATransformer(na=na, dtype=torch.bfloat16)
        gpu.load_state_dict(twin.state_dict())
        gpu = gpu.cuda().eval()
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
            for _ in range(warmup):
                out = gpu(xd)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                out = gpu(xd)
            torch.cuda.synchronize()
            rates[na] = (time.perf_counter() - t0) / steps
    sec = rates["fused_qkv"]
    res = {"model": "PCF-NAT 4x4", "batch": batch, "frames": frames, "dtype": "bf16", "steps": steps,
           "attention": "fused_qkv", "ms_per_batch": round(sec * 1e3, 3), "embeddings_per_s": round(batch / sec, 1)}
    if "fused" in rates:
        res["embeddings_per_s_with_head_copies"] = round(batch / rates["fused"], 1)
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
        threads = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(threads)
        nb = 16
        with torch.no_grad():
            ref = twin(x[:nb])
            t0 = time.perf_counter()
            ref = twin(x[:nb])
            csec = time.perf_counter() - t0
        cos = torch.nn.functional.cosine_similarity(out[:nb].float().cpu(), ref, dim=-1).min().item()
        res["cpu_baseline"] = {"embeddings_per_s": round(nb / csec, 2), "cores": threads, "kind": "port",
                               "sample": "batch %d of %d, one timed pass after one warm-up, PyTorch CPU fp32" % (nb, batch)}
        res["min_cosine_vs_cpu_twin"] = round(cos, 5)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-model", action="store_true", help="skip the PCF-NAT 4x4 embeddings/s leg")
    ap.add_argument("--model-only", action="store_true", help="run only the PCF-NAT 4x4 leg and print its record")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the op shards over "
              "batch*heads with no exchange between GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from na1d_amd import _lib
    from oracle import na1d_oracle as O

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    _lib.load()
    if args.model_only:
        print(json.dumps(model_inference(cpu=not args.no_cpu_baseline, modes=("fused_qkv",))))
        return
    dev = torch.device("cuda:0")
    w = WORKLOADS[args.workload]
    H, T, C, W = w["H"], w["T"], w["C"], w["W"]
    B = w["N"] * H
    _, L = O.split_window(W)
    fwd_bytes, bwd_bytes = algorithmic_bytes(w)
    set_bytes = fwd_bytes + bwd_bytes
    n_sets = max(2, int(600e6 // set_bytes) + 1)      # > 2x the 256 MB Infinity Cache in rotation
    sets = make_sets(w, n_sets, dev)

    # argument tuples are bound once, so that the timed loop is one ctypes call per kernel
    import ctypes
    lib = _lib.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tag = _lib.dtype_tag(sets[0]["q"].dtype)
    fwd_args = [(P(s["o"]), P(s["lse"]), P(s["q"]), P(s["k"]), P(s["v"]), P(s["rpb"]), None, B, H, T, C, W, L, 1.0,
                 tag, stream) for s in sets]
    bwd_args = [(P(s["dq"]), P(s["dk"]), P(s["dv"]), P(s["drpb"]), P(s["q"]), P(s["k"]), P(s["v"]), P(s["o"]),
                 P(s["do"]), P(s["lse"]), P(s["rpb"]), None, B, H, T, C, W, L, 1.0, tag, None, 0, stream)
                for s in sets] if w["bwd"] else None

    def fwd(i):
        _lib.check(lib.na1d_fused_forward(*fwd_args[i % n_sets]), "na1d_fused_forward")

    def bwd(i):
        _lib.check(lib.na1d_fused_backward(*bwd_args[i % n_sets]), "na1d_fused_backward")

    for i in range(max(args.warmup, 1)):
        fwd(i)
        if w["bwd"]:
            bwd(i)
    torch.cuda.synchronize()

    # timed region: exactly K steps between two synchronisations, nothing else in the stream
    K = args.steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(K):
        fwd(i)
        if w["bwd"]:
            bwd(i)
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    ms_per_step = sec / K * 1e3

    # the same K steps again, every launch bracketed by its own pair of HIP events that the library records
    # tightly around the kernel (na1d_profile_events -> hipExtLaunchKernel: the dispatch's begin and end on the
    # launch stream, the interval a profiler's kernel trace reports, without the gaps between launches)
    hip = ctypes.CDLL("libamdhip64.so")

    def new_event():
        e = ctypes.c_void_p()
        assert hip.hipEventCreate(ctypes.byref(e)) == 0
        return e

    def elapsed_ms(a, b):
        ms = ctypes.c_float()
        assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        return ms.value

    pairs = [[(new_event(), new_event()) for _ in range(2)] for _ in range(K)]
    for i in range(K):
        lib.na1d_profile_events(*pairs[i][0])
        fwd(i)
        if w["bwd"]:
            lib.na1d_profile_events(*pairs[i][1])
            bwd(i)
    lib.na1d_profile_events(None, None)
    torch.cuda.synchronize()
    fwd_ms = statistics.mean(elapsed_ms(*p[0]) for p in pairs)
    bwd_ms = statistics.mean(elapsed_ms(*p[1]) for p in pairs) if w["bwd"] else None
    for p in pairs:
        for a, b in p:
            hip.hipEventDestroy(a)
            hip.hipEventDestroy(b)

    # for comparison: K back-to-back launches of the dominant kernel between two stream events (this average
    # includes the gap between consecutive launches)
    dom = bwd if w["bwd"] else fwd
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(K):
        dom(i)
    e1.record()
    torch.cuda.synchronize()
    back_to_back_ms = e0.elapsed_time(e1) / K
    dom_ms = bwd_ms if w["bwd"] else fwd_ms

    value = set_bytes / (sec / K) / 1e9
    if w["bwd"]:
        dom_name, dom_bytes = "fused backward", bwd_bytes
    else:
        dom_name, dom_bytes = "fused forward", fwd_bytes
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
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "kernel": dom_name, "kernel_ms": round(dom_ms, 5), "algorithmic_bytes": dom_bytes},
        "kernels_ms_in_step": {"fused_forward": round(fwd_ms, 5),
                               "fused_backward": None if bwd_ms is None else round(bwd_ms, 5),
                               "dominant_back_to_back_incl_gaps": round(back_to_back_ms, 5)},
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(w)
    if not args.no_model:
        del sets
        torch.cuda.empty_cache()
        try:
            line["pcf_nat_4x4_inference"] = model_inference(cpu=not args.no_cpu_baseline)
        except Exception as e:      # the operator's line above stands on its own
            line["pcf_nat_4x4_inference"] = {"error": "%s: %s" % (type(e).__name__, str(e)[:300])}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
