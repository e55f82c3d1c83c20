#!/usr/bin/env python3
"""Benchmark of the HDLA rank-2 DPLR delta-rule hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload train|fwd|varlen|decode|copy|hdla|hdla_decode|norm|layer|layer_decode] [--no-cpu-baseline]

Default workload ("train") is the headline configuration: chunked forward + backward at B=4, T=2048, H=16,
K=V=64, bf16 inputs, fp32 state, random fp32 initial state, upstream gradients do and dht (configuration 2).
One step = one forward + one backward through the public operator (autograd Function -> C ABI -> HIP kernels)
with all inputs already resident in HBM.  The script prints ONE JSON line: whole-step throughput, a roofline
object for the kernel that takes the largest share of the step (every kernel is listed under "kernels"), and the
CPU oracle timed on this box's host cores on a bounded sample.

Per-kernel durations are measured live with events on the stream the kernels run on, in a second loop of the
same number of steps that launches the same kernels one at a time through hdla_chunk_stages.

Other workloads: fwd (configuration 1), varlen (3), decode (4); copy (the streaming kernel: counter calibration and
attainable HBM rates); hdla, hdla_decode (the operators with a, b formed in the kernels, against building a, b in
torch); norm (gated RMS norm forward + backward); layer, layer_decode (the whole HDLA_Custom layer).
"""
import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "hdla-impl_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
METRIC = "chunked fwd+bwd tokens/s (B4,T2048,H16,K=V=64 bf16) + % of MFMA/HBM roofline"


def _args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # Defaults: the clocks of an idle device take some tens of steps of this length to settle (measured: 0.39 ms a step
    # over steps 6 .. 35 of a fresh process, 0.354 over steps 51 .. 250), so the untimed part is long enough for that
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="train", choices=["train", "fwd", "varlen", "decode", "copy", "hdla", "hdla_decode", "norm", "layer", "layer_decode", "shapes"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--brief", action="store_true", help="the named workload only: no other configurations, no keep_forward "
                    "variant (what the profiler runs recorded under profiles/ use)")
    return ap.parse_args()


def interface_bytes(kernel, pass_, K, V, es, gs, frac_seg=0.0):
    """Algorithmic HBM bytes of one kernel per (16-token chunk, head): every distinct input read once, every
    output written once (es = bytes per element of the inputs, gs = bytes per element of gk)."""
    W, UT, KGT, BGT, VTT, EGL = 32 * K * es, 32 * V * es, 16 * K * es, 32 * K * es, 16 * V * es, 4 * K
    QG, AQK, AQB = 16 * K * es, 256 * es, 512 * es
    AQBT, QGT, TM = 512 * es, 16 * K * es, 1024 * es
    HC = DHC = K * V * es
    DVN = 32 * V * es
    inputs = 2 * 16 * K * es + 16 * K * gs + 2 * 32 * K * es + 16 * V * es          # q,k,gk,a,b,v
    if kernel == "prep":
        out = W + UT + KGT + BGT + VTT + EGL + ((QG + AQK + AQB) if pass_ == 0 else (AQBT + QGT + TM))
        return inputs + out
    if kernel == "scan_fwd":
        rd = W + UT + KGT + BGT + VTT + EGL
        return rd + (QG + AQK + AQB + 16 * V * es if pass_ == 0 else HC)
    if kernel == "scan_bwd":
        return AQBT + W + BGT + QGT + EGL + 16 * V * es + DHC + DVN
    if kernel == "scan_pair":           # both scans of the backward pass in one launch; w, bg and the decay feed both
        return interface_bytes("scan_fwd", 1, K, V, es, gs) + interface_bytes("scan_bwd", 1, K, V, es, gs) - (W + BGT + EGL)
    if kernel == "chunk_grad":
        outs = 2 * 16 * K * es + 16 * K * gs + 2 * 32 * K * es + 16 * V * es
        # (w and u themselves are not read: the kernel rebuilds them from TM, a and v, for the plain operator with decays in
        # the inputs' type)
        return inputs + 16 * V * es + TM + HC + DHC + DVN + outs
    # fused route: the scans' operands stay in LDS.  frac_seg = share of the chunks that lie in segments > 0 (their local
    # output rows, fp32, and the 16 x K block G go through the workspace to the kernel that chains the segments)
    if kernel == "fused_fwd":
        return inputs + (1 - frac_seg) * 16 * V * es + frac_seg * (16 * V * 4 + 16 * K * es)
    if kernel == "fixup":
        return frac_seg * (16 * V * 4 + 16 * K * es + 16 * V * es)
    if kernel == "fused_ckpt":
        return inputs + 16 * V * es + HC + TM
    if kernel == "fused_sum":
        return inputs
    if kernel == "fused_rev":
        return inputs - 16 * V * es + 16 * V * es + DHC + DVN          # q, k, gk, a, b and do in; dS checkpoint and dv_new out
    raise ValueError(kernel)


def algorithmic_bytes(kernel, pass_, K, V, es, gs):
    """Compulsory HBM bytes per (16-token chunk, head) that the roofline fraction is priced on: what the ALGORITHM has
    to move, whatever this implementation's split into kernels writes in between.
      prep, chunk_grad (the kernels that touch the operator's inputs and outputs): the compulsory bytes of their pass --
        forward: q, k, gk, a, b (2 ranks each), v read, o written = (7K + 2V) elements per token and head (9 D at K = V = D);
        backward: the same inputs and do read, dq, dk, dgk, da, db, dv written = (14K + 3V) elements (17 D);
      state scans: per chunk kg (C K), v (C V), w and bg (2 ranks: 4 C K), u (2 C V) read, v_new (2 C V) and the state
        checkpoint (K V) written = C (5K + 5V) elements + K V; the reverse scan likewise (qg, do, w, bg, dv in; dv2, dh out);
        the forward pass's scan writes the output rows instead of a checkpoint and reads qg: C (6K + 4V) elements."""
    C = 16
    if kernel in ("prep", "chunk_grad"):
        if pass_ == 0:
            return C * ((6 * K + 2 * V) * es + K * gs)
        return C * ((12 * K + 3 * V) * es + 2 * K * gs)
    if kernel == "scan_fwd":
        return C * (6 * K + 4 * V) * es if pass_ == 0 else C * (5 * K + 5 * V) * es + K * V * es
    if kernel == "scan_bwd":
        return C * (5 * K + 5 * V) * es + K * V * es
    if kernel == "scan_pair":
        return 2 * (C * (5 * K + 5 * V) * es + K * V * es)
    # fused route: a kernel that prepares and scans is priced on the operator's inputs it must read and on what the
    # algorithm makes it leave behind: the output rows (forward), one state checkpoint per chunk (checkpoint kernel; the
    # reverse kernel also dv_new); the kernel that chains the segments has no compulsory bytes at all
    if kernel == "fused_fwd":
        return C * ((6 * K + 2 * V) * es + K * gs)
    if kernel == "fused_ckpt":
        return C * ((6 * K + 2 * V) * es + K * gs) + K * V * es
    if kernel == "fused_rev":
        return C * ((6 * K + V) * es + K * gs) + K * V * es + 2 * C * V * es
    if kernel == "fused_sum":
        return C * ((6 * K + V) * es + K * gs)
    if kernel == "fixup":
        return 0
    raise ValueError(kernel)


def kernel_sources_digest():
    """Digest of the HIP sources (comments and white space left out, so that only a change of the code changes it): the
    counter summaries under profiles/ record the one they were taken with."""
    import glob
    import hashlib
    import re
    h = hashlib.sha256()
    for f in sorted(glob.glob(os.path.join(ROOT, "hdla-impl_amd", "csrc", "*.*"))):
        if f.endswith((".hip", ".cuh", ".h", ".inc")):
            text = open(f, encoding="utf-8").read()
            text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
            text = re.sub(r"//[^\n]*", " ", text)
            h.update(os.path.basename(f).encode() + b"\0" + " ".join(text.split()).encode() + b"\0")
    return h.hexdigest()[:16]


def traffic_is_current():
    """True when profiles/hbm_traffic.json was collected from the kernels as they are now, False when the sources
    changed since, None when the file does not say."""
    try:
        rec = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json"))).get("kernel_sources_digest")
    except (OSError, ValueError):
        return None
    return None if rec is None else rec == kernel_sources_digest()


def measured_traffic(workload, kernel_key, K, V):
    """HBM bytes per launch of one kernel from the committed rocprofv3 counter summary (profiles/hbm_traffic.json:
    FETCH_SIZE and WRITE_SIZE per dispatch, each scaled by what the same counter reads for the streaming kernel of known traffic), or
    None when that summary does not cover the kernel.  The counters cannot be collected from inside this script."""
    try:
        # the forward-only workload runs the forward kernels of the training step on the same shape
        table = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json"))).get("train" if workload == "fwd" else workload, {})
    except (OSError, ValueError):
        return None
    pass_, name = kernel_key.split(".") if "." in kernel_key else ("", kernel_key)
    fused_mode = {"fused_fwd": "0", "summary": "1", "fused_ckpt": "2", "fused_rev": "3"}.get(name)
    for k, rec in table.items():
        targs = [a.strip() for a in k[k.index("<") + 1:k.rindex(">")].split(",")] if "<" in k else []
        if fused_mode is not None or name == "fixup":
            # fused_kernel<T, GKF32, K, V, MODE (0 forward, 1 summary, 2 checkpoint, 3 reverse), HD>, fixup_kernel<T, K, V>
            if name == "fixup" and k.startswith("fixup_kernel<") and targs[1:3] == [str(K), str(V)]:
                return rec["hbm_bytes_per_launch"]
            if fused_mode is not None and k.startswith("fused_kernel<") and targs[2:] == [str(K), str(V), fused_mode, "false"]:
                return rec["hbm_bytes_per_launch"]
            continue
        if not k.startswith(name + "_kernel<"):
            continue
        # prep<T, GKF32, K, V, MODE (0 forward, 1 backward, 2 kept forward), HD>, scan_fwd<T, K, V, NWC, WRITE_O>, scan_pair<T, K, V, NWC>,
        # chunk_grad<T, GKF32, K, V, HD>, recurrent<T, K, V, BV, HD>
        kv = targs[2:4] if name in ("prep", "chunk_grad") else targs[1:3]
        if kv != [str(K), str(V)]:
            continue
        if name == "prep" and (targs[4] != ("1" if pass_ == "bwd" else "0") or targs[5:] == ["true"]):
            continue
        if name == "scan_fwd" and (targs[4] == "true") != (pass_ == "fwd"):
            continue
        if name in ("chunk_grad", "recurrent") and targs[4:] == ["true"]:
            continue
        return rec["hbm_bytes_per_launch"]
    return None


def norm_traffic(rows):
    """HBM bytes of one backward call of the gated norm at `rows` rows (backward kernel + weight-gradient reduction)
    from the committed counter summary, or None."""
    try:
        table = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json"))).get("norm", {})
        return sum(table[f"{k}@{rows}rows"]["hbm_bytes_per_launch"] for k in ("normalize_bwd_kernel<bf16, 2>", "normalize_dw_kernel"))
    except (OSError, ValueError, KeyError):
        return None


def layer_kernel_times(dev, steps):
    """Event timing of single C-ABI calls of the layer's elementwise and weight-gradient kernels: the pre kernels
    (q | k | v | beta column ranges of a [rows, 3216] projection output, 16 heads of 64), logsigmoid over [rows, 1024]
    and the weight gradient dW [1024, 64] = dY^T X0.  Algorithmic bytes: every input read once, every output written
    once."""
    import ctypes
    from hdla_hip import _lib
    lib = _lib.load()
    P, stream = _lib.ptr, _lib.current_stream(dev)
    H, D, ldy = 16, 64, 3216
    hd = H * D
    res = {}
    for tag, rows in (("config2", 8192), ("hbm", 262144)):
        bf = lambda *shape: torch.randn(*shape, device=dev, dtype=torch.bfloat16)
        y, dy = bf(rows, ldy), torch.empty(rows, ldy, device=dev, dtype=torch.bfloat16)
        q, k, v, beta = bf(rows, hd), bf(rows, hd), bf(rows, hd), bf(rows, H)
        f, lf = bf(rows, hd), torch.empty(rows, hd, device=dev, dtype=torch.bfloat16)
        x0, dw = bf(rows, 2 * D)[:, :D], torch.empty(hd, D, device=dev, dtype=torch.bfloat16)
        dims = _lib.HdlaPreDims(rows, H, D, 0, ldy, 0, hd, 2 * hd, 3 * hd, 0, 1, 0, 2.0, 1e-5)
        nws = lib.hdla_skinny_wgrad_workspace_bytes(0, rows, D, hd)
        ws = torch.empty(nws, dtype=torch.uint8, device=dev)
        cols = (3 * hd + H) * 2
        calls = {
            "layer_pre_fwd": (lambda: lib.hdla_layer_pre_fwd(ctypes.byref(dims), P(y), P(q), P(k), P(v), P(beta), stream),
                              2 * rows * cols),
            "layer_pre_bwd": (lambda: lib.hdla_layer_pre_bwd(ctypes.byref(dims), P(y), P(q), P(k), P(v), P(beta), P(dy), stream),
                              3 * rows * cols),
            "logsigmoid_fwd": (lambda: lib.hdla_logsigmoid_fwd(0, rows * hd, P(f), P(lf), stream), 2 * rows * hd * 2),
            "logsigmoid_bwd": (lambda: lib.hdla_logsigmoid_bwd(0, rows * hd, P(f), P(q), P(lf), stream), 3 * rows * hd * 2),
            "skinny_wgrad": (lambda: lib.hdla_skinny_wgrad(0, rows, D, hd, P(f), hd, P(x0), 2 * D, P(dw), P(ws), nws, stream),
                             rows * (hd + D) * 2 + hd * D * 2),
        }
        for name, (fn, nbytes) in calls.items():
            _lib.check(fn(), name)
            evs = []
            for _ in range(steps):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(); _lib.check(fn(), name); e1.record()
                evs.append((e0, e1))
            torch.cuda.synchronize()
            ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
            res.setdefault(name, {})[tag] = {"rows": rows, "ms": ms, "bytes": nbytes, "GB/s": nbytes / ms / 1e6,
                                             "frac_hbm": nbytes / ms / 1e6 / HBM_PEAK_GBS}
        del y, dy, q, k, v, f, lf, ws
    return res


def time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def stage_times(inp_dev, dims_kw, pass_, steps, outputs):
    """Average duration (ms) of each kernel of one pass, events on the current stream around single-stage launches
    (hdla_chunk_stages).  Classic route: prep, scans, chunk_grad.  Fused route: the forward kernel and the kernel that
    chains the segments (pass 0); checkpoint, reverse and chunk_grad kernels (pass 1), and under the name "summary" what a
    backward pass runs first when the forward pass left no boundary record (not part of the default step)."""
    from hdla_hip import _lib
    lib = _lib.load()
    q, k, v, a, b, gk, h0, do, dht = inp_dev
    dims = _lib.make_dims(**dims_kw)
    ws = _lib.workspace(dims, pass_, q.device)
    P = _lib.ptr
    fused = _lib.workspace_layout(dims, pass_)["ERR"] >= 0
    if fused:
        several = lib.hdla_boundary_bytes(ctypes.byref(dims)) > 0
        names = {2: "fused_fwd", 16: "fixup"} if pass_ == 0 else {16: "summary", 2: "fused_ckpt", 4: "fused_rev", 8: "chunk_grad"}
        masks = ([2, 16] if several else [2]) if pass_ == 0 else (([16] if several else []) + [2, 4, 8])
    else:
        names = {1: "prep", 2: "scan_fwd", 6: "scan_pair", 8: "chunk_grad"}
        masks = [1, 2] if pass_ == 0 else [1, 6, 8]        # the library runs the two backward scans as one launch
    o, ht, dq, dk, dv, da, db, dgk, dh0 = outputs
    stream = _lib.current_stream(q.device)
    acc = {m: 0.0 for m in masks}

    def run(mask):
        rc = lib.hdla_chunk_stages(ctypes.byref(dims), pass_, mask | (1 if fused else 0), P(q), P(k), P(v), P(a), P(b), P(gk),
                                   P(h0), P(o), P(ht), P(do), P(dht), P(dq), P(dk), P(dv), P(da), P(db), P(dgk), P(dh0), P(ws),
                                   ws.numel(), stream)
        _lib.check(rc, "hdla_chunk_stages")

    for m in masks:                      # warm
        run(m)
    torch.cuda.synchronize()
    for _ in range(steps):
        evs = []
        for m in masks:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            run(m)
            e1.record()
            evs.append((m, e0, e1))
        torch.cuda.synchronize()
        for m, e0, e1 in evs:
            acc[m] += e0.elapsed_time(e1)
    return {names[m]: acc[m] / steps for m in masks}


def chunk_table_times(dev, steps=20):
    """Average duration (microseconds) of the kernel that turns cu_seqlens into the chunk table of a packed batch, for 4,
    2048 (the most whose start order is ranked) and 65535 (the most the library takes) sequences of 16 tokens, one head:
    events around launches of that kernel alone (on the fused route stage 1 of hdla_chunk_stages is nothing else)."""
    from hdla_hip import _lib
    lib = _lib.load()
    out = {}
    for N in (4, 2048, 65535):
        T, H, K, V = 16 * N, 1, 64, 64
        cu = (16 * torch.arange(N + 1, dtype=torch.int64)).to(dev)
        dims = _lib.make_dims(1, T, H, K, V, 2, N, torch.bfloat16, torch.bfloat16, 1.0, cu, route=_lib.ROUTE_FUSED)
        ws = _lib.workspace(dims, 0, dev)
        t = [torch.empty(1, T * r, H, K, dtype=torch.bfloat16, device=dev) for r in (1, 1, 1, 2, 2, 1)]
        o = torch.empty(1, T, H, V, dtype=torch.bfloat16, device=dev)
        P, stream = _lib.ptr, _lib.current_stream(dev)

        def run():
            rc = lib.hdla_chunk_stages(ctypes.byref(dims), 0, 1, *[P(x) for x in t], None, P(o), None, *([None] * 9), P(ws),
                                       ws.numel(), stream)
            _lib.check(rc, "hdla_chunk_stages")
        run()
        torch.cuda.synchronize()
        tot = 0.0
        for _ in range(steps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            run()
            e1.record()
            torch.cuda.synchronize()
            tot += e0.elapsed_time(e1)
        out[f"{N} sequences"] = round(tot / steps * 1e3, 1)
        del t, o, ws
    return out


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline_train():
    """The CPU oracle (chunk form of the reference's naive.py, fp32, chunk 16, torch on all host cores), forward + autograd
    backward: one warm-up run and three timed runs (the median is reported) on one batch row of configuration 2 -- every
    (batch, head) is an independent recurrence, so tokens/s does not depend on the rows taken."""
    from hdla_hip.synthetic import make_config
    from oracle import hrdplr_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    inp = make_config(2)
    B_s = 1
    T = inp.q.shape[1]

    def run():
        t = [x[:B_s].bfloat16().float().requires_grad_() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
        h0 = inp.h0[:B_s].clone().requires_grad_()
        t0 = time.perf_counter()
        o, ht = O.chunk_naive(*t, 1.0, h0, chunk_size=16)
        torch.autograd.grad([o, ht], t + [h0], [inp.do[:B_s], inp.dht[:B_s]])
        return time.perf_counter() - t0
    run()
    times = sorted(run() for _ in range(3))
    dt = times[1]
    return {"value": B_s * T / dt, "unit": "tokens/s", "cores": cores, "cpu": cpu_model(), "kind": "port",
            "sample": f"one batch row of configuration 2 (B=1 of 4, T=2048, H=16, K=V=64), fp32 chunk-form oracle fwd + autograd bwd: "
                      f"1 warm-up + 3 timed runs, median {dt:.2f} s (min {times[0]:.2f}, max {times[2]:.2f})"}


def cpu_baseline_decode():
    from hdla_hip.synthetic import make_config
    from oracle import hrdplr_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    steps, B_s = 4, 32
    inp = make_config(4, shape=(B_s, steps, 32, 128, 128))
    t = [x.bfloat16().float() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    t0 = time.perf_counter()
    with torch.no_grad():
        O.recurrence(*t, 1.0, inp.h0, dtype=torch.float32)
    dt = time.perf_counter() - t0
    return {"value": B_s * steps / dt, "unit": "tokens/s", "cores": cores, "cpu": cpu_model(), "kind": "port",
            "sample": f"{steps} decode steps of {B_s} of the 256 sequences (H=32, K=V=128), fp32 token recurrence, {dt:.1f} s"}


def main():
    args = _args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    from hdla_hip import chunk_hrdplr_delta_rule, fused_recurrent_dplr_delta_rule
    from hdla_hip.synthetic import CONFIG_SHAPES, make_config
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    wl = args.workload
    if wl == "shapes":
        # not a benchmark configuration: the chunked forward + backward step over a range of shapes (bf16 inputs, fp32
        # state, h0/do/dht given), default route and keep_forward, to show where the operator stands away from the
        # headline shape (few heads: the scans are a serial chain per head; many: everything is bound by memory)
        shapes = [(4, 2048, 16, 64, 64), (16, 512, 16, 64, 64), (64, 256, 16, 64, 64), (32, 1024, 16, 64, 64), (8, 2048, 32, 64, 64),
                  (1, 8192, 16, 64, 64), (2, 2048, 8, 64, 64), (1, 65536, 2, 64, 64), (4, 2048, 16, 64, 128), (4, 2048, 16, 128, 64),
                  (4, 2048, 16, 128, 128), (8, 2048, 32, 128, 128), (1, 16384, 16, 128, 128)]
        from hdla_hip.synthetic import make_inputs
        rows = []
        for (B, T, H, K, V) in shapes:
            inp = make_inputs(1, B, T, H, K, V)
            leaves = [x.bfloat16().to(dev).requires_grad_(True) for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
            h0 = inp.h0.to(dev).requires_grad_(True)
            do, dht = inp.do.bfloat16().to(dev), inp.dht.to(dev)

            def step(keep=False):
                o, ht = chunk_hrdplr_delta_rule(*leaves, 2, scale=1.0, initial_state=h0, output_final_state=True, keep_forward=keep)
                torch.autograd.grad([o, ht], leaves + [h0], [do, dht])
            sec = time_steps(step, args.steps, args.warmup)
            sec_keep = time_steps(lambda: step(True), args.steps, args.warmup)
            compulsory = B * T * H * (13 * (K + V)) * 2          # 26 D elements of 2 bytes per token and head, D = (K + V) / 2
            rows.append({"B": B, "T": T, "H": H, "K": K, "V": V, "ms_per_step": sec * 1e3, "tokens/s": B * T / sec,
                         "whole_step_frac_hbm": compulsory / sec / (HBM_PEAK_GBS * 1e9),
                         "keep_forward_ms_per_step": sec_keep * 1e3})
            del leaves, h0, do, dht, inp
            torch.cuda.empty_cache()
        print(json.dumps({"metric": "chunked fwd+bwd over shapes (bf16)", "steps": args.steps, "warmup": args.warmup, "shapes": rows}))
        return
    if wl == "copy":
        # calibration workload, not a benchmark of the operator: the library's streaming kernel, whose traffic per
        # launch is known exactly (the HBM traffic counters are scaled by what they read for the 1:1 launches,
        # which come last and are the ones timed for "GB/s"), and the rate HBM sustains for several read:write mixes
        import ctypes
        from hdla_hip import _lib
        lib = _lib.load()
        n = 256 << 20
        bufs = [torch.empty(n, dtype=torch.uint8, device=dev).fill_(i + 1) for i in range(6)]
        stream = _lib.current_stream(dev)
        turn = [0]

        def launch(nr, nw):
            # successive launches take different buffers, so that none is served from the 256 MB last-level cache
            turn[0] += 1
            rot = bufs[turn[0] % 6:] + bufs[:turn[0] % 6]
            rd = (ctypes.c_void_p * 3)(*[b.data_ptr() for b in rot[:nr]], *([None] * (3 - nr)))
            wr = (ctypes.c_void_p * 2)(*[b.data_ptr() for b in rot[3:3 + nw]], *([None] * (2 - nw)))
            _lib.check(lib.hdla_calib_stream(rd, nr, wr, nw, n, stream), "hdla_calib_stream")

        mixes = {}
        for nr, nw in ((1, 0), (0, 1), (3, 1), (2, 1), (1, 2), (1, 1)):
            sec = time_steps(lambda: launch(nr, nw), args.steps, args.warmup)
            mixes[f"{nr}:{nw}"] = round((nr + nw) * n / sec / 1e9)
        print(json.dumps({"metric": "copy calibration", "bytes_read_per_launch": n, "bytes_written_per_launch": n,
                          "ms_per_step": sec * 1e3, "GB/s": 2 * n / sec / 1e9, "GB/s_by_read_write_mix": mixes}))
        return
    if wl == "layer_decode":
        # One cached decode step of the whole HDLA_Custom layer on the layer shape of configuration 4: embed_dim =
        # H*K = 4096, 32 heads of 128, 256 sequences, one token each per call, fp32 state carried in the cache.
        from hdla_hip.layer import HDLA_Custom, RecurrentCache
        B, H, D = 256, 32, 128
        d = H * D
        torch.manual_seed(0)
        m = HDLA_Custom(d, H, token_mixer_init_type=2, rescale_type=0).to(dev).bfloat16().eval()
        xs = [torch.randn(B, 1, d, device=dev, dtype=torch.bfloat16) for _ in range(8)]
        st = {"cache": RecurrentCache(), "i": 0}
        with torch.no_grad():
            _, st["cache"] = m(torch.randn(B, 16, d, device=dev, dtype=torch.bfloat16), past_key_values=st["cache"], use_cache=True)

            def step():
                st["i"] += 1
                _, st["cache"] = m(xs[st["i"] % 8], past_key_values=st["cache"], use_cache=True)
            sec = time_steps(step, args.steps, args.warmup)
        state_bytes = 2 * B * H * D * D * 4
        print(json.dumps({"metric": "HDLA layer decode tokens/s", "value": B / sec, "unit": "tokens/s", "n_gpus": 1,
                          "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": True,
                          "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                          "config": {"workload": "HDLA_Custom layer, embed_dim 4096, 32 heads of 128, 256 sequences, one "
                                                 "token per call, state carried in the cache", "batch": B},
                          "roofline": {"bound": "hbm", "kernel": "whole step (recurrent_kernel streams the state; weights 137 MB)",
                                       "achieved": (state_bytes + 137e6) / sec / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                       "frac": (state_bytes + 137e6) / sec / 1e9 / HBM_PEAK_GBS, "traffic": None,
                                       "note": "state read + written once and every weight read once, over the step's wall time"}}))
        return
    if wl == "layer":
        # The whole HDLA token mixer (projections, activations, normalisations, the operator, output gate and
        # projection) on the layer shape of configuration 2: embed_dim = H*K = 1024, 16 heads, B=4, T=2048, bf16
        # parameters; forward + backward (gradients of x and of every parameter).  `value` is the whole step (its GEMMs
        # are the BLAS library's); "layer_kernels" times this library's kernels around the operator one by one through
        # the C ABI, on the step's shape (cache-resident) and on 32x the rows (HBM), like the norm workload.
        from hdla_hip.layer import HDLA_Custom
        B, T, H, D = 4, 2048, 16, 64
        d = H * D
        torch.manual_seed(0)
        x = torch.randn(B, T, d, device=dev, dtype=torch.bfloat16, requires_grad=True)
        do = torch.randn(B, T, d, device=dev, dtype=torch.bfloat16)
        out = {}
        for name, kw in (("fused", {}), ("plain_route", {"fuse_ab": False})):
            m = HDLA_Custom(d, H, token_mixer_init_type=2, rescale_type=0, **kw).to(dev).bfloat16().train()

            params = [p for p in m.parameters()]

            def grads():
                # gradients of x and of every parameter, handed over as new tensors (what an optimizer step that
                # clears gradients with set_to_none sees), not accumulated into existing ones
                y, _ = m(x)
                return [y.detach()] + list(torch.autograd.grad(y, [x] + params, do))
            out[name] = time_steps(grads, args.steps, args.warmup)
            if name == "fused":
                # the same step as one HIP graph (the library only launches kernels, so it can be captured): removes the
                # host's share; every replay is checked against the eager step before it is timed
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    grads()
                torch.cuda.current_stream().wait_stream(side)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    static = grads()
                ref = grads()
                exact = True
                for _ in range(3):
                    graph.replay()
                    torch.cuda.synchronize()
                    grads()                                   # eager work between replays
                    # this library's kernels are deterministic; a BLAS kernel that splits its inner dimension with
                    # atomics may not be, so bit equality is reported and only a real difference is an error
                    exact = exact and all(torch.equal(a, b) for a, b in zip(static, ref))
                    worst = max(float((a.float() - b.float()).norm() / (b.float().norm() + 1e-30)) for a, b in zip(static, ref))
                    if worst > 1e-2:
                        raise RuntimeError(f"graph replay differs from the eager step (relative L2 {worst:.2e})")
                out["fused_graph"] = time_steps(graph.replay, args.steps, args.warmup)
                out["graph_exact"] = exact
                del graph, static, ref
        print(json.dumps({"metric": "HDLA layer fwd+bwd tokens/s", "value": B * T / out["fused"], "unit": "tokens/s",
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": out["fused"] * 1e3,
                          "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
                          "data": "synthetic",
                          "config": {"workload": "HDLA_Custom layer, embed_dim 1024, 16 heads of 64, B=4 T=2048, bf16; "
                                                 "forward + backward", "global_batch": B, "seq_len": T},
                          "as_hip_graph": {"what": "the same forward + backward captured once and replayed (replays checked against the eager step)",
                                           "ms_per_step": out["fused_graph"] * 1e3, "value": B * T / out["fused_graph"],
                                           "replays_bit_equal_to_eager": out["graph_exact"]},
                          "plain_route": {"what": "same layer with fuse_ab=False: torch parameterize_a_b + the plain operator",
                                          "ms_per_step": out["plain_route"] * 1e3, "value": B * T / out["plain_route"]},
                          "layer_kernels": layer_kernel_times(dev, args.steps),
                          "roofline": None}))
        return
    if wl == "norm":
        # The gated RMS norm the HDLA layer applies to the operator's output (hdla_custom.py:341-345), forward +
        # backward, on the layer's shape for configuration 2 (B*T = 8192 rows of H*V = 1024 channels, bf16; the five
        # tensors of the backward pass are 80 MiB together and stay in the last-level cache) and on 32x the rows,
        # which is what HBM sees; the roofline entry is the backward kernel on the large shape.
        from hdla_hip.normalize import normalize_fn
        g = torch.Generator().manual_seed(0)
        out = {}
        for name, rows in (("config2", 8192), ("hbm", 262144)):
            D = 1024
            x = torch.randn(rows, D, generator=g).bfloat16().to(dev).requires_grad_()
            gate = torch.randn(rows, D, generator=g).bfloat16().to(dev).requires_grad_()
            w = torch.ones(D, device=dev, requires_grad=True)
            do = torch.randn(rows, D, generator=g).bfloat16().to(dev)
            res = {}

            def fwd():
                res["o"] = normalize_fn(x, w, gate=gate, gate_pos="pre", c=D ** 0.5, eps=1e-5)

            def bwd():
                torch.autograd.grad(res["o"], [x, gate, w], do, retain_graph=True)

            def both():
                fwd()
                torch.autograd.grad(res["o"], [x, gate, w], do)
            sec = time_steps(both, args.steps, args.warmup)
            # the two passes by themselves: C entry points on preallocated tensors, events on the launch stream
            import ctypes
            from hdla_hip import _lib
            lib = _lib.load()
            dims = _lib.HdlaNormDims(rows, 1, D, 0, 1, 1, D ** 0.5, 1e-5)
            o, dx, dg = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
            dw = torch.empty(D, dtype=torch.float32, device=dev)
            nws = lib.hdla_normalize_workspace_bytes(ctypes.byref(dims))
            ws = torch.empty(nws, dtype=torch.uint8, device=dev)
            P, stream = _lib.ptr, _lib.current_stream(dev)

            def fwd_c():
                _lib.check(lib.hdla_normalize_fwd(ctypes.byref(dims), P(x), P(w), P(gate), P(o), stream), "hdla_normalize_fwd")

            def bwd_c():
                _lib.check(lib.hdla_normalize_bwd(ctypes.byref(dims), P(x), P(w), P(gate), P(do), P(dx), P(dg), P(dw),
                                                  P(ws), nws, stream), "hdla_normalize_bwd")
            ms = {}
            for nm, fn in (("fwd", fwd_c), ("bwd", bwd_c)):
                fn()
                evs = []
                for _ in range(args.steps):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(); fn(); e1.record()
                    evs.append((e0, e1))
                torch.cuda.synchronize()
                ms[nm] = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
            del o, dx, dg, ws
            nb = {"fwd": 3 * rows * D * 2 + D * 4, "bwd": 5 * rows * D * 2 + D * 8}
            out[name] = {"rows": rows, "channels": D, "ms_per_step": sec * 1e3, "rows/s": rows / sec,
                         "fwd_ms": ms["fwd"], "bwd_ms": ms["bwd"], "fwd_bytes": nb["fwd"], "bwd_bytes": nb["bwd"],
                         "fwd_GB/s": nb["fwd"] / ms["fwd"] / 1e6, "bwd_GB/s": nb["bwd"] / ms["bwd"] / 1e6}
            del x, gate, do, res
        big = out["hbm"]
        line = {"metric": "gated rms norm fwd+bwd rows/s", "value": out["config2"]["rows/s"], "unit": "rows/s", "n_gpus": 1,
                "steps": args.steps, "warmup": args.warmup, "ms_per_step": out["config2"]["ms_per_step"],
                "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                "config": {"workload": "gated RMS norm of the layer at configuration 2's shape: 8192 rows x 1024 channels, "
                                       "bf16 tensors, fp32 weight, gate before the norm; forward + backward"},
                "shapes": out,
                "roofline": {"bound": "hbm", "kernel": "normalize_bwd_kernel (+ normalize_dw_kernel), 262144 rows",
                             "achieved": big["bwd_GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": big["bwd_GB/s"] / HBM_PEAK_GBS, "traffic": norm_traffic(262144),
                             "bytes_per_launch": big["bwd_bytes"], "ms_per_launch": big["bwd_ms"],
                             "note": "one call of hdla_normalize_bwd: the backward kernel and the small weight-gradient reduction after it"}}
        if not args.no_cpu_baseline:
            from oracle import normalize_oracle as NO
            cores = os.cpu_count() or 1
            torch.set_num_threads(cores)
            rows = 8192
            xc = torch.randn(rows, 1024, generator=g).bfloat16().float().requires_grad_()
            gc_ = torch.randn(rows, 1024, generator=g).bfloat16().float().requires_grad_()
            wc = torch.ones(1024, requires_grad=True)
            t0 = time.perf_counter()
            reps = 5
            for _ in range(reps):
                o = NO.rms_norm_fused_gate(xc, gc_, wc, dtype=torch.float32)
                torch.autograd.grad(o, [xc, gc_, wc], torch.ones_like(o))
            dtc = (time.perf_counter() - t0) / reps
            line["cpu_baseline"] = {"value": rows / dtc, "unit": "rows/s", "cores": cores, "kind": "port",
                                    "sample": f"{reps} runs of the config-2 shape (8192 x 1024), fp32 torch oracle fwd + autograd bwd"}
        print(json.dumps(line))
        return
    cfg = {"train": 2, "fwd": 1, "varlen": 3, "decode": 4, "hdla": 2, "hdla_decode": 4}[wl]
    B, T, H, K, V = CONFIG_SHAPES[cfg]
    inp = make_config(cfg) if wl in ("hdla", "hdla_decode") else None
    dt = torch.bfloat16
    res = {"metric": METRIC if wl == "train" else f"{wl} tokens/s", "unit": "tokens/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "bf16", "data": "synthetic"}

    if wl == "decode":
        res.update(run_decode_workload(args.steps, args.warmup, dev))
        if not args.no_cpu_baseline:
            res["cpu_baseline"] = cpu_baseline_decode()
        print(json.dumps(res))
        return

    if wl == "hdla_decode":
        # One decode step of the HDLA layer on the shape of configuration 4: a and b formed per token inside the
        # token-serial kernel, against the layer's own route (torch builds a, b from beta, k, log_f, then the plain
        # recurrent operator).  Whole-step rates only; the kernel's traffic is the state, as for "decode".
        from hdla_hip import fused_recurrent_hdla_delta_rule, parameterize_a_b
        from hdla_hip.synthetic import make_inputs
        ncycle = 8
        gen = [inp] + [make_inputs(2000 + i, B, 1, H, K, V, h0_std=0.1) for i in range(1, ncycle)]
        g = torch.Generator().manual_seed(0)
        steps_in = [[x.to(dt).to(dev) for x in (c.q, c.k, c.v, 2.0 * torch.rand(B, 1, H, 1, generator=g), c.gk)] for c in gen]
        state = {"S": inp.h0.to(dev), "i": 0}

        def fused():
            t = steps_in[state["i"] % ncycle]
            state["i"] += 1
            _, state["S"] = fused_recurrent_hdla_delta_rule(*t, scale=1.0, initial_state=state["S"], output_final_state=True)

        def plain():
            q, k, v, beta, lf = steps_in[state["i"] % ncycle]
            state["i"] += 1
            a, b = parameterize_a_b(beta.float(), k.float(), lf.float())
            _, state["S"] = fused_recurrent_dplr_delta_rule(q, k, v, a.to(dt), b.to(dt), lf, 2, scale=1.0,
                                                            initial_state=state["S"], output_final_state=True)

        sec = time_steps(fused, args.steps, args.warmup)
        state["S"] = inp.h0.to(dev)
        sec_plain = time_steps(plain, args.steps, args.warmup)
        nbytes = 2 * B * H * K * V * 4 + B * H * (3 * K + V + V + 1) * 2
        res.update(metric="decode tokens/s with a, b given by (beta, k, log_f)", value=B / sec, ms_per_step=sec * 1e3,
                   config={"workload": "configuration 4 shape (B=256 H=32 K=V=128, one token per call, persistent fp32 "
                                       "state), a and b formed in the kernel", "batch": B, "heads": H, "K": K, "V": V},
                   plain_route={"what": "torch parameterize_a_b (fp32, eager) + fused_recurrent_dplr_delta_rule",
                                "ms_per_step": sec_plain * 1e3, "value": B / sec_plain},
                   roofline={"bound": "hbm", "kernel": "recurrent_kernel", "achieved": nbytes / sec / 1e9,
                             "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / sec / 1e9 / HBM_PEAK_GBS,
                             "traffic": None, "bytes_per_launch": nbytes, "ms_per_launch": sec * 1e3,
                             "note": "whole step on the host clock (one kernel per step)"})
        print(json.dumps(res))
        return

    if wl == "hdla":
        # The operator as the HDLA layer calls it (a, b given by beta, k, log_f), on the shape of configuration 2:
        # a and b formed inside the kernels against the layer's own route (torch builds a, b, the plain operator runs
        # on them, autograd goes back through both).  Whole-step rates only.
        from hdla_hip import chunk_hdla_delta_rule, parameterize_a_b
        g = torch.Generator().manual_seed(0)
        beta = (2.0 * torch.rand(B, T, H, 1, generator=g)).to(dt).to(dev).requires_grad_()
        q, k, v, lf = [x.to(dt).to(dev).requires_grad_() for x in (inp.q, inp.k, inp.v, inp.gk)]
        h0 = inp.h0.to(dev).requires_grad_()
        do, dht = inp.do.to(dt).to(dev), inp.dht.to(dev)

        def fused():
            o, ht = chunk_hdla_delta_rule(q, k, v, beta, lf, scale=1.0, initial_state=h0, output_final_state=True)
            torch.autograd.grad([o, ht], [q, k, v, beta, lf, h0], [do, dht])

        def plain():
            a, b = parameterize_a_b(beta.float(), k.float(), lf.float())
            o, ht = chunk_hrdplr_delta_rule(q, k, v, a.to(dt), b.to(dt), lf, 2, scale=1.0, initial_state=h0,
                                            output_final_state=True, chunk_size=16)
            torch.autograd.grad([o, ht], [q, k, v, beta, lf, h0], [do, dht])

        sec = time_steps(fused, args.steps, args.warmup)
        sec_plain = time_steps(plain, args.steps, args.warmup)
        res.update(metric="chunked fwd+bwd tokens/s with a, b given by (beta, k, log_f)", value=B * T / sec,
                   ms_per_step=sec * 1e3,
                   config={"workload": "configuration 2 shape (B=4 T=2048 H=16 K=V=64, bf16), a and b formed in the kernels",
                           "global_batch": B, "seq_len": T, "heads": H, "K": K, "V": V, "chunk": 16},
                   plain_route={"what": "torch parameterize_a_b (fp32, eager) + chunk_hrdplr_delta_rule + autograd through both",
                                "ms_per_step": sec_plain * 1e3, "value": B * T / sec_plain},
                   roofline=None)
        print(json.dumps(res))
        return
    res.update(run_chunk_workload(wl, cfg, args.steps, args.warmup, dev, keep_variant=not args.brief))
    if wl == "train" and not args.brief:
        # the other configurations, measured in this process after the headline (fewer steps: they are reported, the
        # headline is what the step count is about)
        n_other = max(5, args.steps // 3)
        others = {}
        for name, owl, ocfg in (("config1_fwd", "fwd", 1), ("config3_varlen", "varlen", 3)):
            r = run_chunk_workload(owl, ocfg, n_other, max(3, args.warmup // 3), dev)
            others[name] = {"workload": r["config"]["workload"], "tokens/s": r["value"], "ms_per_step": r["ms_per_step"],
                            "dominant_kernel": r["roofline"]["kernel"], "frac": r["roofline"]["frac"],
                            "achieved_GB/s": r["roofline"]["achieved"], "traffic": r["roofline"]["traffic"],
                            "whole_step_frac_hbm": r["whole_step"]["frac_hbm"],
                            **({"keep_forward": r["keep_forward"]} if "keep_forward" in r else {}),
                            "kernels": [{k: x[k] for k in ("kernel", "ms", "frac_hbm", "frac_interface")} for x in r["kernels"]]}
        r = run_decode_workload(4 * n_other, max(5, args.warmup), dev)
        others["config4_decode"] = {"workload": r["config"]["workload"], "tokens/s": r["value"], "ms_per_step": r["ms_per_step"],
                                    "dominant_kernel": "recurrent_kernel", "frac": r["roofline"]["frac"],
                                    "achieved_GB/s": r["roofline"]["achieved"], "traffic": r["roofline"]["traffic"],
                                    "ms_per_launch": r["roofline"]["ms_per_launch"]}
        res["other_configs"] = others
        res["chunk_table_us"] = chunk_table_times(dev)
    if not args.no_cpu_baseline and wl == "train":
        res["cpu_baseline"] = cpu_baseline_train()
    print(json.dumps(res))


def run_chunk_workload(wl, cfg, steps, warmup, dev, keep_variant=True):
    """One of the chunked configurations (train = 2, fwd = 1, varlen = 3): whole-step time through the public operator,
    then every kernel by itself."""
    from hdla_hip import chunk_hrdplr_delta_rule
    from hdla_hip.synthetic import CONFIG_SHAPES, make_config
    B, T, H, K, V = CONFIG_SHAPES[cfg]
    inp = make_config(cfg)
    dt = torch.bfloat16
    cu = None if inp.cu_seqlens is None else inp.cu_seqlens.to(dev)
    N = B if cu is None else cu.numel() - 1
    leaves = [x.to(dt).to(dev).requires_grad_(wl != "fwd") for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    use_h0 = wl != "fwd"
    h0 = inp.h0.to(dev).requires_grad_(True) if use_h0 else None
    do, dht = inp.do.to(dt).to(dev), inp.dht.to(dev)

    def step(keep=False):
        o, ht = chunk_hrdplr_delta_rule(*leaves, 2, scale=1.0, initial_state=h0, output_final_state=True,
                                        chunk_size=16, cu_seqlens=cu, keep_forward=keep)
        if wl != "fwd":
            torch.autograd.grad([o, ht], leaves + [h0], [do, dht])

    sec = time_steps(step, steps, warmup)
    # the same step on the other routes the library has for this shape (reported beside `value`, never as it): strictly
    # the inputs kept between the passes (the fused route's default hands the states at the time-segment boundaries, 64 KiB
    # per sequence, head and segment, from the forward to the backward pass; without them the backward pass re-derives
    # them with one more pass over the inputs), and the classic launch plan (separate prep and scan kernels)
    variants = {}
    if keep_variant:
        from hdla_hip import _lib as _l
        probe = _l.make_dims(B, T, H, K, V, 2, N, dt, dt, 1.0, cu)
        if _l.load().hdla_boundary_bytes(ctypes.byref(probe)) > 0 and wl != "fwd":
            os.environ["HDLA_HIP_INPUTS_ONLY"] = "1"
            variants["inputs_only"] = time_steps(step, steps, warmup)
            del os.environ["HDLA_HIP_INPUTS_ONLY"]
        if _l.workspace_layout(probe, 0)["ERR"] >= 0:
            os.environ["HDLA_HIP_ROUTE"] = "classic"
            variants["classic_route"] = time_steps(step, steps, warmup)
            del os.environ["HDLA_HIP_ROUTE"]
    # the same step with keep_forward=True (an option, off by default: the forward pass's per-chunk intermediates stay
    # alive until the backward pass, which then does not recompute them); `value` is the default route
    sec_keep = time_steps(lambda: step(True), steps, warmup) if wl != "fwd" and keep_variant else None
    tokens = B * T
    # per-kernel durations
    raw = [x.detach() for x in leaves] + [None if h0 is None else h0.detach(), do, dht]
    dims_kw = dict(B=B, T=T, H=H, K=K, V=V, R=2, N=N, in_dtype=dt, gk_dtype=dt, scale=1.0, cu_seqlens=cu)
    o = torch.empty_like(raw[2])
    ht = torch.empty(N, H, K, V, dtype=torch.float32, device=dev)
    grads = [torch.empty_like(x) for x in (raw[0], raw[1], raw[2], raw[3], raw[4], raw[5])]
    dh0 = torch.empty_like(ht)
    outs = (o, ht, *grads, dh0)
    kern = {}
    for pass_ in ([0] if wl == "fwd" else [0, 1]):
        for name, ms in stage_times(raw, dims_kw, pass_, steps, outs).items():
            kern[f"{'fwd' if pass_ == 0 else 'bwd'}.{name}"] = ms
    nchunk_heads = H * sum(-(-int(l) // 16) for l in ([T] * B if cu is None else (cu[1:] - cu[:-1]).tolist()))
    from hdla_hip import _lib as _l
    probe = _l.make_dims(B, T, H, K, V, 2, N, dt, dt, 1.0, cu)
    nseg = max(1, _l.load().hdla_boundary_bytes(ctypes.byref(probe)) // (N * H * K * V * 4))
    frac_seg = (nseg - 1) / nseg                           # share of the chunks in time segments other than the first
    summary_ms = kern.pop("bwd.summary", None)             # only a backward pass without a boundary record runs it
    klist = []
    for name, ms in kern.items():
        p_, kn = name.split(".")
        alg = algorithmic_bytes(kn, 0 if p_ == "fwd" else 1, K, V, 2, 2) * nchunk_heads
        itf = interface_bytes(kn, 0 if p_ == "fwd" else 1, K, V, 2, 2, frac_seg) * nchunk_heads
        klist.append({"kernel": name, "ms": ms, "bytes": alg, "GB/s": alg / (ms * 1e-3) / 1e9,
                      "frac_hbm": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                      "interface_bytes": itf, "frac_interface": itf / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                      "traffic": measured_traffic(wl, name, K, V)})
    dom = max(klist, key=lambda x: x["ms"])
    per_tok_head = ((7 * K + 2 * V) * 2) if wl == "fwd" else ((21 * K + 5 * V) * 2)   # compulsory bytes per (token, head)
    whole = per_tok_head * H * tokens
    keep = {} if sec_keep is None else {"keep_forward": {
        "what": "the same step with keep_forward=True: the backward pass reads the forward pass's per-chunk intermediates "
                "instead of recomputing them (more memory held between the passes than the reference's inputs-only contract)",
        "ms_per_step": sec_keep * 1e3, "value": tokens / sec_keep,
        "whole_step_frac_hbm": ((21 * K + 5 * V) * 2) * H * tokens / sec_keep / 1e9 / HBM_PEAK_GBS}}
    other = {}
    if "inputs_only" in variants:
        other["inputs_only"] = {
            "what": "the same step with HDLA_HIP_INPUTS_ONLY=1: nothing but the inputs kept between the passes; the backward "
                    "pass re-derives the states at the time-segment boundaries with one more pass (kernel time under summary_ms)",
            "ms_per_step": variants["inputs_only"] * 1e3, "value": tokens / variants["inputs_only"], "summary_ms": summary_ms}
    if "classic_route" in variants:
        other["classic_route"] = {"what": "the same step with HDLA_HIP_ROUTE=classic: prep, scan and chunk_grad kernels with the "
                                          "scans' operands passed through the workspace",
                                  "ms_per_step": variants["classic_route"] * 1e3, "value": tokens / variants["classic_route"]}
    return dict(
        **keep, **other,
        route="fused" if any("fused" in x["kernel"] for x in klist) else "classic", time_segments=nseg,
        value=tokens / sec, ms_per_step=sec * 1e3,
        config={"workload": {"train": "config 2: chunked fwd+bwd, B=4 T=2048 H=16 K=V=64, bf16 in, fp32 state, h0/do/dht",
                             "fwd": "config 1: chunked fwd, B=4 T=2048 H=16 K=V=64, bf16 in, fp32 state",
                             "varlen": "config 3: chunked fwd+bwd, packed 2048/4096/4096/6144, H=16 K=V=128"}[wl],
                "global_batch": B, "seq_len": T, "heads": H, "K": K, "V": V, "chunk": 16},
        roofline={"bound": "hbm", "kernel": dom["kernel"], "achieved": dom["GB/s"], "peak": HBM_PEAK_GBS,
                  "unit": "GB/s", "frac": dom["frac_hbm"],
                  "traffic": measured_traffic(wl, dom["kernel"], K, V),
                  "traffic_from_current_kernels": traffic_is_current(),
                  "bytes_per_launch": dom["bytes"], "ms_per_launch": dom["ms"],
                  "note": "achieved = compulsory bytes of the kernel's pass (every input of the operator read once, every "
                          "output written once; for the scans their operands and one state checkpoint per chunk) over the "
                          "kernel's time; frac_interface in `kernels` counts what this implementation's kernels hand each "
                          "other as well; traffic = HBM bytes per launch from the committed counter summary"},
        kernels=klist,
        whole_step={"compulsory_bytes": whole, "GB/s": whole / sec / 1e9, "frac_hbm": whole / sec / 1e9 / HBM_PEAK_GBS,
                    "sum_kernel_ms": sum(x["ms"] for x in klist)})


def run_decode_workload(steps, warmup, dev):
    """Configuration 4: one token per call for 256 sequences, the fp32 state carried from call to call."""
    from hdla_hip import fused_recurrent_dplr_delta_rule
    from hdla_hip.recurrent import fused_recurrent_dplr_delta_rule_fwd
    from hdla_hip.synthetic import CONFIG_SHAPES, make_config, make_inputs
    B, T, H, K, V = CONFIG_SHAPES[4]
    inp = make_config(4)
    dt = torch.bfloat16
    ncycle = 8                                             # distinct per-step inputs, cycled
    gen = [inp] + [make_inputs(2000 + i, B, 1, H, K, V, h0_std=0.1) for i in range(1, ncycle)]
    steps_in = [[x.to(dt).to(dev) for x in (g.q, g.k, g.v, g.a, g.b, g.gk)] for g in gen]
    state = {"S": inp.h0.to(dev), "i": 0}

    def step():
        t = steps_in[state["i"] % ncycle]
        state["i"] += 1
        _, state["S"] = fused_recurrent_dplr_delta_rule(*t, 2, scale=1.0, initial_state=state["S"],
                                                        output_final_state=True)
    sec = time_steps(step, steps, warmup)
    # kernel-only duration with events on the launch stream
    evs = []
    for _ in range(steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t = steps_in[state["i"] % ncycle]
        state["i"] += 1
        q, k, v, a, b, gk = t
        e0.record()
        _, state["S"] = fused_recurrent_dplr_delta_rule_fwd(q, k, v, a, b, gk, 2, 1.0, state["S"], True)
        e1.record()
        evs.append((e0, e1))
    torch.cuda.synchronize()
    kms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    nbytes = 2 * B * H * K * V * 4 + B * H * (4 * K + 4 * K + V + V) * 2
    return dict(value=B / sec, ms_per_step=sec * 1e3,
                config={"workload": "config 4: fused recurrent decode, B=256 H=32 K=V=128, one token per call, "
                                    "persistent fp32 state", "batch": B, "heads": H, "K": K, "V": V},
                roofline={"bound": "hbm", "kernel": "recurrent_kernel", "achieved": nbytes / (kms * 1e-3) / 1e9,
                          "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / (kms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                          "traffic": measured_traffic("decode", "recurrent", K, V),
                          "traffic_from_current_kernels": traffic_is_current(),
                          "bytes_per_launch": nbytes, "ms_per_launch": kms})


if __name__ == "__main__":
    main()
