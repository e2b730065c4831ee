#!/usr/bin/env python3
"""Benchmark of the Forgetting Attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4|c5|decode|c3d64|c3d32|c3d16|shift|norm_gate|ref_sweep|acp_sweep|power]
                    [--no-extras] [--no-cpu-baseline]

A step is one forward + backward pass of ``forgetting_attention`` over one batch
of synthetic input already resident in HBM (forward only for c5).  The default
workload is the long-context training-layer shape (B=4, T=16384, H=16, D=128,
bf16, gate logits ~ N(3,1), head_first=False, no pruning); its FLOP count uses the
reference's convention, fwd+bwd = 7*B*H*T^2*D.  One JSON line is printed.

Besides the headline value the line carries
  roofline     : the dominant kernel (dK/dV) timed alone with events on the launch
                 stream, against the bf16 MFMA peak;
  kernels      : the same for every stage of the path;
  cpu_baseline : the PyTorch fp32 restatement of the reference's materialised-mask
                 attention on this host's cores: forward + backward (autograd) of one
                 (batch, head) pair of config 3, best of two runs of about 7 s each, and
                 the forward of config 1;
  backward_credited_frac : the five matrix products the FLOP convention credits to the
                 backward over the time of its two kernels, against the peak (the split
                 backward executes seven);
  acp          : pruned-tile fraction and speed-up of Adaptive Computation Pruning
                 (thresholds "auto" and -10.0) on strongly decaying gates;
  prefill      : chunked-prefill shape (M=128, N=32768, left padding), HBM GB/s;
  decode       : one new token against the same cache;
  head_dim_*   : the headline step at head dims 64, 32 and 16 (same token count and matmul work);
  library_example : the small B4 T512 H12 D64 step, wall time against the sum of its kernels.
--workload ref_sweep runs the reference's own benchmark recipe (its __main__ block) instead.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "forgetting-transformer_amd"))
sys.path.insert(0, str(ROOT))


def power_sampler(csv_path, stop_path, period_s=0.02):
    """Child process of --workload power: polls the SMI library for socket power, shader clock, temperature and
    throttle status until `stop_path` appears; one CSV line per sample, stamped with time.time().  Never touches HIP."""
    import amdsmi
    amdsmi.amdsmi_init()
    dev = amdsmi.amdsmi_get_processor_handles()[0]

    def num(x):
        try:
            return float(x)
        except (TypeError, ValueError):
            return float("nan")

    with open(csv_path, "w") as f:
        try:
            cap = amdsmi.amdsmi_get_power_cap_info(dev)
        except Exception as e:   # noqa: BLE001 -- the sampler reports what the library offers on this box
            cap = {"error": repr(e)}
        f.write("# power_cap_info " + json.dumps({k: str(v) for k, v in cap.items()}) + "\n")
        f.write("t,socket_w,gfx_mhz,gfx_mhz_max,hotspot_c,throttle\n")
        first = True
        while not os.path.exists(stop_path):
            t = time.time()
            try:
                m = amdsmi.amdsmi_get_gpu_metrics_info(dev)
            except Exception as e:   # noqa: BLE001
                f.write(f"# metrics error {e!r}\n")
                break
            if first:
                f.write("# first sample keys " + json.dumps(sorted(m.keys())) + "\n")
                first = False
            clks = [num(c) for c in (m.get("current_gfxclks") or []) if num(c) == num(c) and 0 < num(c) < 60000]
            w = num(m.get("current_socket_power"))
            if not w == w or w <= 0 or w > 60000:
                w = num(m.get("average_socket_power"))
            mhz = sum(clks) / len(clks) if clks else num(m.get("current_gfxclk"))
            f.write(f"{t:.4f},{w:.1f},{mhz:.1f},{max(clks) if clks else mhz:.1f},{num(m.get('temperature_hotspot')):.1f},"
                    f"{m.get('throttle_status')}\n")
            f.flush()
            dt = period_s - (time.time() - t)
            if dt > 0:
                time.sleep(dt)
    amdsmi.amdsmi_shut_down()


if len(sys.argv) == 4 and sys.argv[1] == "--power-sampler":   # before torch is imported: the sampler needs none of it
    power_sampler(sys.argv[2], sys.argv[3])
    sys.exit(0)

import torch  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0

# HBM bytes per launch of the dominant kernel of a workload (fetched + written) come from two rocprofv3 --pmc
# passes over this script (FETCH_SIZE, WRITE_SIZE; counters cannot be read from inside the timed run).  The
# summary of those passes, profiles/hbm_traffic_c3_c5.md, ends with a machine-readable block: the bytes per
# workload and the SHA-256 of the kernel sources they were measured on.  measured_traffic() returns the figure
# only while those sources are unchanged; otherwise the roofline carries traffic = null and says why.
TRAFFIC_PROFILE = ROOT / "profiles" / "hbm_traffic_c3_c5.md"
KERNEL_SOURCES = ["fox_common.hpp", "fox_kernels.hpp", "fox_fwd.hip", "fox_bwd.hip", "fox_decode.hip"]


def kernel_source_digest():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        h.update((ROOT / "forgetting-transformer_amd" / "csrc" / name).read_bytes())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    """(bytes per launch or None, provenance string)."""
    import re
    if not TRAFFIC_PROFILE.exists():
        return None, "no HBM traffic profile committed"
    m = re.search(r"```json traffic\n(.*?)\n```", TRAFFIC_PROFILE.read_text(), flags=re.S)
    if not m:
        return None, f"{TRAFFIC_PROFILE.name} has no traffic block"
    block = json.loads(m.group(1))
    rel = f"profiles/{TRAFFIC_PROFILE.name}"
    if workload not in block["bytes_per_launch"]:
        return None, f"{rel} has no entry for {workload}"
    if block["kernel_source_digest"] != kernel_source_digest():
        return None, (f"{rel} was measured on kernel sources {block['kernel_source_digest']}, the tree holds "
                      f"{kernel_source_digest()}: re-run its two rocprofv3 --pmc passes")
    return float(block["bytes_per_launch"][workload]), f"{rel} (kernel sources {block['kernel_source_digest']})"


WORKLOADS = {
    # name: B, T(M), N, H, D, gate mean, gate std, head_first, fwd_only, seq_start
    "c2": dict(B=4, M=512, N=512, H=12, D=64, mean=0.0, std=1.0, head_first=False, fwd_only=False, pad=False),
    # config 3 at the other head dims: same token count and matmul work, the heads scaled up
    "c3d32": dict(B=4, M=16384, N=16384, H=64, D=32, mean=3.0, std=1.0, head_first=False, fwd_only=False, pad=False),
    "c3d16": dict(B=4, M=16384, N=16384, H=128, D=16, mean=3.0, std=1.0, head_first=False, fwd_only=False, pad=False),
    "c3": dict(B=4, M=16384, N=16384, H=16, D=128, mean=3.0, std=1.0, head_first=False, fwd_only=False, pad=False),
    # config 3 at the head dim of the reference's own models (hidden_size / num_heads = 64 in every
    # configs/experiment/longcrawl64/forgetting_transformer/*.yaml): same token count and matmul work, twice the heads
    "c3d64": dict(B=4, M=16384, N=16384, H=32, D=64, mean=3.0, std=1.0, head_first=False, fwd_only=False, pad=False),
    "c4": dict(B=4, M=16384, N=16384, H=16, D=128, mean=-1.0, std=2.0, head_first=False, fwd_only=False, pad=False),
    "c5": dict(B=16, M=128, N=32768, H=16, D=128, mean=2.0, std=1.0, head_first=True, fwd_only=True, pad=True),
    # one new token against the same cache (the reference's M == 1 path, ops/forgetting_attention.py:148-153)
    "decode": dict(B=16, M=1, N=32768, H=16, D=128, mean=2.0, std=1.0, head_first=True, fwd_only=True, pad=True),
}


def synth(w, device, seed=0):
    """Synthetic inputs of a workload, generated on the device from a fixed seed."""
    g = torch.Generator(device=device).manual_seed(seed)
    B, M, N, H, D = w["B"], w["M"], w["N"], w["H"], w["D"]
    shape_q = (B, H, M, D) if w["head_first"] else (B, M, H, D)
    shape_k = (B, H, N, D) if w["head_first"] else (B, N, H, D)
    shape_g = (B, H, N) if w["head_first"] else (B, N, H)
    q = torch.randn(shape_q, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    k = torch.randn(shape_k, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    v = torch.randn(shape_k, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    logits = torch.randn(shape_g, generator=g, device=device, dtype=torch.float32) * w["std"] + w["mean"]
    log_fgate = torch.nn.functional.logsigmoid(logits)
    dout = torch.randn(shape_q, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    seq_start = None
    if w["pad"]:
        seq_start = torch.randint(0, 8192, (B,), generator=g, device=device, dtype=torch.long)
    return q, k, v, log_fgate, dout, seq_start


def flops_fwd(w):
    # causal with offset: sum over rows of (row + P_SEQ + 1) columns, 4*D flops per (row, column)
    M, N = w["M"], w["N"]
    pairs = M * (N - M) + M * (M + 1) / 2
    return 4.0 * w["B"] * w["H"] * pairs * w["D"]


def time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def event_time(fn, iters, warmup=2):
    """Average duration (s) of ``fn`` measured with events on the current stream."""
    for _ in range(warmup):
        fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) * 1e-3 / iters


def stage_times(w, tensors, iters, threshold=None):
    """Time every kernel of the path alone through the C ABI (launches go to torch's current stream).
    threshold: optional pruning threshold, a float applied to every (batch, head) or a (B, H) fp32 tensor."""
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import _view

    lib = _lib.load()
    q, k, v, log_fgate, dout, seq_start = tensors
    if not w["head_first"]:
        q, k, v, dout = (x.transpose(1, 2) for x in (q, k, v, dout))
        log_fgate = log_fgate.transpose(1, 2)
    B, H, M, D = q.shape
    N = k.shape[2]
    dev = q.device
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    dims = _lib.Dims(B, H, M, N, D, _lib.DTYPE_BF16)
    c = torch.empty((B, H, N), dtype=torch.float32, device=dev)
    lse = torch.empty((B, H, M), dtype=torch.float32, device=dev)
    o = torch.empty_like(q)
    ss = None if seq_start is None else seq_start.data_ptr()
    ws_bytes = C.c_int64(0)
    _lib.check(lib.fox_attn_fwd_workspace_bytes(C.byref(dims), C.byref(ws_bytes)), "workspace")
    ws = torch.empty(max(ws_bytes.value, 16), dtype=torch.uint8, device=dev)  # key-split partials (prefill / decode shapes)
    thr = None
    if threshold is not None:
        thr_t = (threshold if torch.is_tensor(threshold)
                 else torch.full((B, H), float(threshold), dtype=torch.float32, device=dev))
        thr = thr_t.data_ptr()
    fwd = _lib.FwdArgs(dims, _view(q), _view(k), _view(v), _view(o), c.data_ptr(), lse.data_ptr(), ss, thr,
                       1.0 / math.sqrt(D), None, ws.data_ptr() if ws_bytes.value else None, ws_bytes.value)
    out = {}

    def scan():
        _lib.check(lib.fox_cumsum_fwd(log_fgate.data_ptr(), *log_fgate.stride(), ss, c.data_ptr(), B, H, N, stream), "scan")

    def f():
        _lib.check(lib.fox_attn_fwd(C.byref(fwd), stream), "fwd")

    # the same prologue from bf16 gate logits with logsigmoid fused in (forgetting_attention_from_logits)
    logits = torch.randn(log_fgate.shape, device=dev).bfloat16()
    if not w["head_first"]:
        logits = logits.transpose(1, 2).contiguous().transpose(1, 2)
    lg = torch.empty_like(c)

    def gate_scan():
        _lib.check(lib.fox_gate_cumsum_fwd(logits.data_ptr(), _lib.DTYPE_BF16, *logits.stride(), ss, lg.data_ptr(), c.data_ptr(),
                                           B, H, N, stream), "gate scan")

    gate_scan()
    out["gate_cumsum_fwd"] = event_time(gate_scan, iters)
    out["torch_logsigmoid"] = event_time(lambda: torch.nn.functional.logsigmoid(logits.float()), iters)
    scan()
    out["cumsum_fwd"] = event_time(scan, iters)
    out["fwd"] = event_time(f, iters)
    if w["fwd_only"]:
        return out
    delta = torch.empty((2,) + tuple(lse.shape), dtype=torch.float32, device=dev)
    dc = torch.empty_like(c)
    dg = torch.empty_like(c)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    bwd = _lib.BwdArgs(dims, _view(q), _view(k), _view(v), _view(o), _view(dout), _view(dq), _view(dk), _view(dv),
                       c.data_ptr(), lse.data_ptr(), ss, thr, 1.0 / math.sqrt(D), delta[0].data_ptr(), delta[1].data_ptr(),
                       dc.data_ptr(), dg.data_ptr())
    for name, fn in (("bwd_dq", lib.fox_attn_bwd_dq), ("bwd_dkdv", lib.fox_attn_bwd_dkdv)):
        out[name] = event_time(lambda fn=fn, name=name: _lib.check(fn(C.byref(bwd), stream), name), iters)
    out["cumsum_bwd"] = event_time(
        lambda: _lib.check(lib.fox_cumsum_bwd(dc.data_ptr(), dg.data_ptr(), 0, 0, 0, None, B, H, N, stream), "cumsum_bwd"), iters)
    return out


def cpu_baseline(budget_s=5.0):
    """The reference's pure-PyTorch path (restated in oracle/) on the host cores.  `value`: forward + backward of a
    bounded sample of the benchmark's own workload, one (batch, head) pair of config 3 (T = 16384, D = 128, fp32,
    materialised 1 GiB score matrix, gradients through autograd), in the metric's FLOP convention.  `config1_forward`:
    the forward of the configuration the reference's pure-PyTorch path is meant for (B2 T256 H4 D64)."""
    from oracle.fox_oracle import forgetting_attention_ref, forgetting_attention_ref_grads

    def same_workload_sample():
        w = WORKLOADS["c3"]
        T, D = w["N"], w["D"]
        g = torch.Generator().manual_seed(1)
        q, k, v, do = (torch.randn((1, T, 1, D), generator=g) for _ in range(4))
        lf = torch.nn.functional.logsigmoid(torch.randn((1, T, 1), generator=g) * w["std"] + w["mean"])
        times = []
        for _ in range(2):   # the first run also pays for the allocator's first touch of ~8 GiB
            t0 = time.perf_counter()
            forgetting_attention_ref_grads(q, k, v, lf, do)
            times.append(time.perf_counter() - t0)
        sec = min(times)
        return 7.0 * T * T * D / sec * 1e-12, sec, T, D

    tflops, sec, T3, D3 = same_workload_sample()

    B, T, H, D = 2, 256, 4, 64
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn((B, T, H, D), generator=g) for _ in range(3))
    log_fgate = torch.nn.functional.logsigmoid(torch.randn((B, T, H), generator=g))
    cores = torch.get_num_threads()
    fn = lambda: forgetting_attention_ref(q, k, v, log_fgate, sm_scale=1.0 / math.sqrt(D))
    for _ in range(3):
        fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while time.perf_counter() < t_end and len(times) < 2000:
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    flops = 4.0 * B * H * (T * (T + 1) / 2) * D
    return {
        "value": tflops, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"oracle/fox_oracle.py forward + backward (autograd), fp32, one (batch, head) pair of config 3 "
                  f"(1 of 64: T{T3} D{D3}), best of 2 runs ({sec:.2f} s), FLOPs 7*T^2*D as in `value`",
        "config1_forward": {
            "value": flops / med * 1e-12, "unit": "TFLOP/s",
            "sample": f"oracle/fox_oracle.py forward, fp32, B{B} T{T} H{H} D{D}, median of {len(times)} runs "
                      f"({med * 1e3:.3f} ms), causal FLOPs 4*B*H*T(T+1)/2*D"},
    }


def graph_time(step, steps):
    """Seconds per step of `step` captured once into a HIP graph and replayed: the same kernels without the host
    between them (allocation, Python, launch latency), which matters when the whole step is about a millisecond."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up off the capture stream, as autograd under capture requires
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def kept_fraction(start_index, M, N, block_m, block_n):
    """Share of causal (query block, key block) tiles the forward visits, from the kernel's own bounds."""
    p_seq = N - M
    n_mt = start_index.shape[-1]
    m0 = torch.arange(n_mt, device=start_index.device) * block_m
    hi = torch.clamp(p_seq + m0 + block_m, max=N)
    total = ((hi + block_n - 1) // block_n).sum().item() * start_index.shape[0] * start_index.shape[1]
    kept = (((hi + block_n - 1) // block_n)[None, None, :] - start_index // block_n).sum().item()
    return kept / total


def acp_report(steps, warmup):
    from forgetting_transformer import forgetting_attention
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import ForgettingAttention

    w = WORKLOADS["c4"]
    q, k, v, log_fgate, dout, _ = synth(w, "cuda", seed=1)
    q, k, v, log_fgate = (x.requires_grad_() for x in (q, k, v, log_fgate))
    block_m, block_n, _, _ = _lib.tile_config(w["D"])
    rep = {"workload": "B4 T16384 H16 D128 bf16 fwd+bwd, gate logits N(-1, 2)"}
    base = None
    ref_out = None
    for name, thr in (("none", None), ("auto", "auto"), ("-10.0", -10.0)):
        def step():
            out = forgetting_attention(q, k, v, log_fgate, adaptive_threshold=thr)
            out.backward(dout)
            q.grad = k.grad = v.grad = log_fgate.grad = None
        t = time_steps(step, steps, warmup)
        t_graph = graph_time(step, max(steps, 10))
        with torch.no_grad():
            out = forgetting_attention(q, k, v, log_fgate, adaptive_threshold=thr)
        entry = {"ms_per_step": t * 1e3, "graph_replay_ms_per_step": t_graph * 1e3}
        if thr is None:
            base, base_graph, ref_out = t, t_graph, out
        else:
            with torch.no_grad():
                _, _, si = ForgettingAttention.apply(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                                     log_fgate.transpose(1, 2), None, True, None, thr, False, True)
            kept = kept_fraction(si, w["M"], w["N"], block_m, block_n)
            entry.update(pruned_tile_fraction=1.0 - kept, speedup_vs_none=base / t,
                         graph_replay_speedup_vs_none=base_graph / t_graph,
                         max_abs_diff_vs_none=(out.float() - ref_out.float()).abs().max().item())
        rep[name] = entry
    # where the pruned step spends its time: every kernel alone at threshold -10, against the bytes it must move
    q, k, v, log_fgate = (x.detach() for x in (q, k, v, log_fgate))
    st = stage_times(w, (q, k, v, log_fgate, dout, None), max(3, steps), threshold=-10.0)
    S, R = w["B"] * w["H"] * w["M"] * w["D"] * 2, w["B"] * w["H"] * w["M"] * 4
    alg = {"fwd": 4 * S + 2 * R, "bwd_dq": 6 * S + 5 * R, "bwd_dkdv": 6 * S + 6 * R}
    rep["pruned_kernels"] = {k_: {"ms": st[k_] * 1e3, "algorithmic_gbps": alg[k_] / st[k_] * 1e-9} for k_ in alg}
    return rep


def prefill_report(steps, warmup):
    from forgetting_transformer import forgetting_attention

    w = WORKLOADS["c5"]
    sets = [synth(w, "cuda", seed=10 + i) for i in range(3)]  # rotate so K/V do not sit in cache
    idx = [0]

    def step():
        q, k, v, log_fgate, _, ss = sets[idx[0] % len(sets)]
        idx[0] += 1
        with torch.no_grad():
            forgetting_attention(q, k, v, log_fgate, head_first=True, seq_start=ss)
    t = time_steps(step, steps, warmup)
    B, H, M, N, D = w["B"], w["H"], w["M"], w["N"], w["D"]
    pad = torch.stack([s[5] for s in sets]).float().mean(0)  # mean left padding per batch row over the rotated sets
    kv_bytes = (2.0 * H * (N - pad) * D * 2).sum().item()
    other = 2 * B * H * M * D * 2 + B * H * N * 4 * 2
    return {"workload": "B16 M128 N32768 H16 D128 bf16 forward, head_first, seq_start~U[0,8192)",
            "ms_per_step": t * 1e3, "algorithmic_bytes": kv_bytes + other, "hbm_gbps": (kv_bytes + other) / t * 1e-9,
            "frac_of_8TBps": (kv_bytes + other) / t * 1e-9 / PEAK_HBM_GBPS}


def decode_report(steps, warmup):
    """One new token against the config-5 cache (M = 1): the streaming kernel, HBM-bound."""
    from forgetting_transformer import forgetting_attention

    w = WORKLOADS["decode"]
    sets = [synth(w, "cuda", seed=20 + i) for i in range(3)]  # rotate so K/V do not sit in cache
    idx = [0]

    def step():
        q, k, v, log_fgate, _, ss = sets[idx[0] % len(sets)]
        idx[0] += 1
        with torch.no_grad():
            forgetting_attention(q, k, v, log_fgate, head_first=True, seq_start=ss)
    t = time_steps(step, steps, warmup)
    st = stage_times(w, sets[0], max(5, steps))
    B, H, M, N, D = w["B"], w["H"], w["M"], w["N"], w["D"]
    pad = sets[0][5].float()
    alg = (2.0 * H * (N - pad) * D * 2).sum().item() + 2 * B * H * M * D * 2 + B * H * N * 4
    out = {"workload": "B16 M1 N32768 H16 D128 bf16 forward, head_first, seq_start~U[0,8192)",
           "ms_per_step": t * 1e3, "kernel_ms": st["fwd"] * 1e3, "algorithmic_bytes": alg,
           "kernel_hbm_gbps": alg / st["fwd"] * 1e-9, "kernel_frac_of_8TBps": alg / st["fwd"] * 1e-9 / PEAK_HBM_GBPS}

    # The step as the layer runs it while generating: append the new token's key, value and gate to the cache, then
    # attend.  The cache that grows in place copies the new token only; the reference's cache concatenates
    # (fgate_cache.py:107-116), i.e. re-copies the layer's whole cache at every token.
    from forgetting_transformer import FgateDynamicCache
    q, k, v, log_fgate, _, ss = sets[0]
    del sets
    torch.cuda.empty_cache()
    n0 = N - 64
    k1, v1, g1 = k[:, :, n0:n0 + 1], v[:, :, n0:n0 + 1], log_fgate[:, :, n0:n0 + 1]
    cache = FgateDynamicCache(max_length=N)
    cache.update(k[:, :, :n0], v[:, :, :n0], log_fgate[:, :, :n0], 0)

    def step_in_place():
        cache.crop(n0)                       # the same position every time, so that all timed steps are alike
        kk, vv, gg = cache.update(k1, v1, g1, 0)
        forgetting_attention(q, kk, vv, gg, head_first=True, seq_start=ss)

    state = [k[:, :, :n0].contiguous(), v[:, :, :n0].contiguous(), log_fgate[:, :, :n0].contiguous()]

    def step_concatenating():
        kk, vv, gg = torch.cat([state[0], k1], dim=2), torch.cat([state[1], v1], dim=2), torch.cat([state[2], g1], dim=2)
        forgetting_attention(q, kk, vv, gg, head_first=True, seq_start=ss)

    with torch.no_grad():
        out["ms_per_step_with_cache_append"] = time_steps(step_in_place, steps, warmup) * 1e3
        out["ms_per_step_with_concatenating_cache"] = time_steps(step_concatenating, steps, warmup) * 1e3
    return out


def head_dim_report(steps, warmup, name="c3d64"):
    """The headline step at another head dim, same token count and matmul work as the D = 128 workload: 64 (what
    every model configuration of the reference uses: configs/experiment/longcrawl64/forgetting_transformer/*.yaml
    have hidden_size / num_heads = 64), 32 and 16 (the remaining tile specialisations)."""
    from forgetting_transformer import forgetting_attention

    w = WORKLOADS[name]
    tensors = synth(w, "cuda")
    q, k, v, log_fgate, dout, _ = tensors
    q, k, v, log_fgate = (x.requires_grad_() for x in (q, k, v, log_fgate))

    def step():
        forgetting_attention(q, k, v, log_fgate, head_first=w["head_first"]).backward(dout)
        q.grad = k.grad = v.grad = log_fgate.grad = None
    t = time_steps(step, steps, warmup)
    st = stage_times(w, tensors, max(3, steps))
    unit = flops_fwd(w) / 2.0
    rep = {"workload": f"B{w['B']} T{w['M']} H{w['H']} D{w['D']} bf16 fwd+bwd, gate logits N({w['mean']},{w['std']}), no pruning",
           "ms_per_step": t * 1e3, "tflops": 7 * unit / t * 1e-12, "frac_of_bf16_peak": 7 * unit / t * 1e-12 / PEAK_BF16_TFLOPS,
           "kernels": {name: {"ms": st[name] * 1e3, "tflops": m * unit / st[name] * 1e-12}
                       for name, m in (("fwd", 2), ("bwd_dkdv", 4), ("bwd_dq", 3))}}
    return rep


def small_shape_report(steps, warmup):
    """The library-example shape (B4 T512 H12 D64 bf16 fwd+bwd): launch-latency-bound.  Wall time per step of the
    operator (Python, autograd, allocations, launches), the same step replayed from a HIP graph, and the sum of
    its kernels timed alone."""
    from forgetting_transformer import forgetting_attention

    w = WORKLOADS["c2"]
    tensors = synth(w, "cuda", seed=2)
    q, k, v, log_fgate, dout, _ = tensors
    q, k, v, log_fgate = (x.requires_grad_() for x in (q, k, v, log_fgate))

    def step():
        forgetting_attention(q, k, v, log_fgate).backward(dout)
        q.grad = k.grad = v.grad = log_fgate.grad = None
    t = time_steps(step, max(steps, 300), max(warmup, 30))
    t_graph = graph_time(step, max(steps, 300))
    st = stage_times(w, tensors, max(steps, 20))
    path = ("cumsum_fwd", "fwd", "bwd_dq", "bwd_dkdv", "cumsum_bwd")
    return {"workload": "B4 T512 H12 D64 bf16 fwd+bwd, gate logits N(0,1)", "wall_ms_per_step": t * 1e3,
            "graph_replay_ms_per_step": t_graph * 1e3, "kernel_sum_ms": sum(st[n] for n in path) * 1e3,
            "kernels_ms": {n: st[n] * 1e3 for n in path}}


def ref_sweep_report(ns):
    """The reference's own benchmark recipe (ops/forgetting_attention.py:1438-1513): B4 H32 D64 bf16, head-first,
    N_CTX = 2^10 .. 2^14, gate logits ~ U(0,10), sm_scale = 1.3, threshold -10 per (batch, head); forward and
    backward (o.backward(do, retain_graph=True), gradients accumulating) timed separately like
    triton.testing.do_bench: events around every call, the cache flushed by zeroing a buffer before each, about
    25 ms of warm-up and 100 ms of timed calls, mean.  FLOPs as there: forward 2*B*H*N^2*D (causal), backward
    2.5 x forward.  One JSON line."""
    from forgetting_transformer import forgetting_attention

    B, H, D = 4, 32, 64
    dev = "cuda"
    flush = torch.empty(512 << 20, dtype=torch.int8, device=dev)   # larger than the 256 MiB last-level cache

    def do_bench(fn, warmup_ms=25.0, rep_ms=100.0):
        fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(5):
            flush.zero_()
            fn()
        e.record()
        torch.cuda.synchronize()
        est = s.elapsed_time(e) / 5
        n_warm, n_rep = max(1, int(warmup_ms / est)), max(3, int(rep_ms / est))
        for _ in range(n_warm):
            fn()
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
        for i in range(n_rep):
            flush.zero_()
            starts[i].record()
            fn()
            ends[i].record()
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in zip(starts, ends)) / n_rep

    rows = []
    for n_ctx in [2 ** i for i in range(10, 15)]:
        g = torch.Generator(device=dev).manual_seed(n_ctx)
        q, k, v = (torch.randn((B, H, n_ctx, D), generator=g, device=dev, dtype=torch.float32).bfloat16().requires_grad_()
                   for _ in range(3))
        logit = torch.empty((B, H, n_ctx), dtype=torch.float32, device=dev).uniform_(0, 10, generator=g)
        log_fgate = torch.nn.functional.logsigmoid(logit).requires_grad_()
        thr = torch.full((B, H), -10.0, dtype=torch.float, device=dev)
        fwd = lambda: forgetting_attention(q, k, v, log_fgate, head_first=True, sm_scale=1.3, adaptive_threshold=thr)
        ms_f = do_bench(fwd)
        o = fwd()
        do = torch.randn(o.shape, generator=g, device=dev, dtype=torch.float32).bfloat16()
        ms_b = do_bench(lambda: o.backward(do, retain_graph=True))
        f_fwd = 2.0 * B * H * n_ctx * n_ctx * D     # 2 matmuls x 2*B*H*N^2*D, halved for the causal mask
        rows.append({"N_CTX": n_ctx, "fwd_ms": ms_f, "fwd_tflops": f_fwd / ms_f * 1e-9, "bwd_ms": ms_b,
                     "bwd_tflops": 2.5 * f_fwd / ms_b * 1e-9})
        del q, k, v, log_fgate, o, do
    top = rows[-1]
    total_ms = top["fwd_ms"] + top["bwd_ms"]
    value = 3.5 * 2.0 * B * H * top["N_CTX"] ** 2 * D / total_ms * 1e-9
    print(json.dumps({
        "metric": "reference benchmark recipe: fwd and bwd TFLOP/s over N_CTX (value: fwd+bwd at N_CTX=16384)",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": ns.steps, "warmup": ns.warmup, "ms_per_step": total_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "ref_sweep: B4 H32 D64 bf16 head_first, N_CTX 1024..16384, gate logits U(0,10), sm_scale 1.3, "
                               "adaptive_threshold -10 per (batch, head); ops/forgetting_attention.py:1438-1513",
                   "flops_convention": "fwd 2*B*H*N^2*D, bwd 2.5 x fwd (causal)", "timing": "events per call, cache flushed before "
                   "each call, ~25 ms warm-up, ~100 ms timed, mean (triton.testing.do_bench)"},
        "frac_of_bf16_peak": value / PEAK_BF16_TFLOPS, "sweep": rows}))


def acp_sweep_report(ns):
    """Speed-up of the pruned step against the unpruned one on the same inputs, as a function of how much pruning
    keeps: config 4's shape with constant gates -10/W, so that with adaptive_threshold = -10 every query row keeps a
    band of W keys (W * T - W^2 / 2 of the T^2 / 2 causal pairs).  One JSON line."""
    from forgetting_transformer import forgetting_attention

    w = dict(WORKLOADS["c4"])
    q, k, v, g, do, _ = synth(w, "cuda", seed=1)
    q, k, v = (x.requires_grad_() for x in (q, k, v))
    T = w["N"]
    steps, warmup = max(3, ns.steps // 2), 2

    def step(gates, thr):
        out = forgetting_attention(q, k, v, gates, adaptive_threshold=thr)
        out.backward(do)
        q.grad = k.grad = v.grad = gates.grad = None

    rows = []
    for W in (128, 256, 512, 1024, 2048, 4096, 8192):
        gates = torch.full_like(g, -10.0 / W).requires_grad_()
        t_full = time_steps(lambda: step(gates, None), steps, warmup)
        t_acp = time_steps(lambda: step(gates, -10.0), steps, warmup)
        st = stage_times(w, (q.detach(), k.detach(), v.detach(), gates.detach(), do, None), steps, threshold=-10.0)
        kept = (W * T - W * W / 2.0) / (T * T / 2.0)
        rows.append({"band_keys": W, "kept_fraction": kept, "ms_unpruned": t_full * 1e3, "ms_pruned": t_acp * 1e3,
                     "speedup": t_full / t_acp, "proportional_speedup": 1.0 / kept,
                     "fraction_of_proportional": (t_full / t_acp) * kept,
                     "kernels_ms": {name: st[name] * 1e3 for name in ("fwd", "bwd_dq", "bwd_dkdv")}})
    line = {
        "metric": "ACP speed-up vs no-prune on the same inputs, by kept fraction", "value": rows[0]["speedup"], "unit": "x",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": rows[0]["ms_pruned"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"acp_sweep: B{w['B']} T{T} H{w['H']} D{w['D']} bf16 fwd+bwd, constant gates -10/W, "
                               "adaptive_threshold -10, W = kept band in keys"},
        "sweep": rows,
    }
    print(json.dumps(line))


def shift_report(ns):
    """Token shift (the key/value pre-processing of the FoX layer) at the training-layer shape:
    forward + backward, HBM-bound; one JSON line of its own."""
    from forgetting_transformer import token_shift
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.token_shift import _args

    B, T, H, D = 4, 16384, 16, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(B, T, H, D, generator=g, device="cuda").bfloat16().requires_grad_()
    dout = torch.randn(B, T, H, D, generator=g, device="cuda").bfloat16()
    curr = torch.rand(B, T, H, generator=g, device="cuda").requires_grad_()

    def step():
        out = token_shift(x, 1.0 - curr, curr)
        out.backward(dout)
        x.grad = curr.grad = None
    sec = time_steps(step, ns.steps, ns.warmup)

    lib = _lib.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    xd, cd = x.detach(), curr.detach()
    pd = 1.0 - cd
    out, dx = torch.empty_like(xd), torch.empty_like(xd)
    dp, dc = torch.empty_like(cd), torch.empty_like(cd)
    fwd_args = _args(xd, pd, cd, out=out)
    bwd_args = _args(xd, pd, cd, dout=dout, dx=dx, dprev_weight=dp, dcurr_weight=dc)
    t_f = event_time(lambda: _lib.check(lib.fox_token_shift_fwd(C.byref(fwd_args), stream), "shift fwd"), max(5, ns.steps))
    t_b = event_time(lambda: _lib.check(lib.fox_token_shift_bwd(C.byref(bwd_args), stream), "shift bwd"), max(5, ns.steps))
    S, W = B * T * H * D * 2, B * T * H * 4
    bytes_f, bytes_b = 2 * S + 2 * W, 3 * S + 4 * W
    kernels = {"shift_fwd": {"ms": t_f * 1e3, "gbps": bytes_f / t_f * 1e-9, "algorithmic_bytes": bytes_f},
               "shift_bwd": {"ms": t_b * 1e3, "gbps": bytes_b / t_b * 1e-9, "algorithmic_bytes": bytes_b}}
    value = (bytes_f + bytes_b) / sec * 1e-9
    line = {
        "metric": "token shift fwd+bwd, algorithmic HBM GB/s (operator incl. autograd and the 1 - curr elementwise op)",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": ns.steps, "warmup": ns.warmup, "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"shift: B{B} T{T} H{H} D{D} bf16 fwd+bwd, weights fp32 (B,T,H)"},
        "roofline": {"kernel": "shift_bwd", "bound": "hbm", "achieved": kernels["shift_bwd"]["gbps"], "peak": PEAK_HBM_GBPS,
                     "unit": "GB/s", "frac": kernels["shift_bwd"]["gbps"] / PEAK_HBM_GBPS,
                     "traffic": None, "algorithmic_bytes": bytes_b,
                     "avg_launch_ms": t_b * 1e3},
        "kernels": kernels,
    }
    print(json.dumps(line))


def norm_gate_report(ns):
    """Gated per-head RMS norm (the FoX layer's epilogue on the attention output) at the training-layer
    shape: forward + backward, HBM-bound; one JSON line of its own."""
    from forgetting_transformer import group_norm_gated
    from forgetting_transformer.ops import _lib

    B, T, G, D = 4, 16384, 16, 128
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(B, T, G * D, generator=gen, device="cuda").bfloat16().requires_grad_()
    g = torch.randn(B, T, G * D, generator=gen, device="cuda").bfloat16().requires_grad_()
    dy = torch.randn(B, T, G * D, generator=gen, device="cuda").bfloat16()
    w = (torch.rand(G * D, generator=gen, device="cuda") + 0.5).requires_grad_()

    def step():
        y = group_norm_gated(x, g, w, None, "sigmoid", is_rms_norm=True, num_groups=G)
        y.backward(dy)
        x.grad = g.grad = w.grad = None
    sec = time_steps(step, ns.steps, ns.warmup)

    lib = _lib.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rows, width = B * T, G * D
    xd, gd, wd = x.detach().view(rows, width), g.detach().view(rows, width), w.detach()
    y, dx, dg = torch.empty_like(xd), torch.empty_like(xd), torch.empty_like(xd)
    rstd = torch.empty(rows, G, device="cuda")
    dw = torch.empty(width, device="cuda")
    nb = C.c_int64(0)
    _lib.check(lib.fox_norm_gate_workspace_bytes(rows, G, D, C.byref(nb)), "workspace")
    ws = torch.empty(nb.value, dtype=torch.uint8, device="cuda")
    args = _lib.NormGateArgs(rows, G, D, _lib.DTYPE_BF16, _lib.ACT_SIGMOID, 1e-6, xd.data_ptr(), width, gd.data_ptr(), width,
                             wd.data_ptr(), y.data_ptr(), width, rstd.data_ptr(), dy.data_ptr(), width, dx.data_ptr(), width,
                             dg.data_ptr(), width, dw.data_ptr(), ws.data_ptr())
    t_f = event_time(lambda: _lib.check(lib.fox_norm_gate_fwd(C.byref(args), stream), "norm fwd"), max(5, ns.steps))
    t_b = event_time(lambda: _lib.check(lib.fox_norm_gate_bwd(C.byref(args), stream), "norm bwd"), max(5, ns.steps))
    S = rows * width * 2
    bytes_f, bytes_b = 3 * S + rows * G * 4, 5 * S + rows * G * 4 + 2 * nb.value
    kernels = {"norm_gate_fwd": {"ms": t_f * 1e3, "gbps": bytes_f / t_f * 1e-9, "algorithmic_bytes": bytes_f},
               "norm_gate_bwd": {"ms": t_b * 1e3, "gbps": bytes_b / t_b * 1e-9, "algorithmic_bytes": bytes_b}}
    # the same kernels without a gate: the per-head RMS norm of queries and keys (QK-norm); one tensor less each way
    args.activation, args.g, args.dg = _lib.ACT_NONE, None, None
    t_pf = event_time(lambda: _lib.check(lib.fox_norm_gate_fwd(C.byref(args), stream), "norm fwd"), max(5, ns.steps))
    t_pb = event_time(lambda: _lib.check(lib.fox_norm_gate_bwd(C.byref(args), stream), "norm bwd"), max(5, ns.steps))
    bytes_pf, bytes_pb = 2 * S + rows * G * 4, 3 * S + rows * G * 4 + 2 * nb.value
    kernels["qk_norm_fwd"] = {"ms": t_pf * 1e3, "gbps": bytes_pf / t_pf * 1e-9, "algorithmic_bytes": bytes_pf}
    kernels["qk_norm_bwd"] = {"ms": t_pb * 1e3, "gbps": bytes_pb / t_pb * 1e-9, "algorithmic_bytes": bytes_pb}
    # The same norm applied in the epilogue of the attention forward (forgetting_attention_norm_gate), against the
    # forward followed by the norm kernel, without pruning and with 97.7 % of the tiles pruned (config 4's gates).
    from forgetting_transformer import forgetting_attention, forgetting_attention_norm_gate
    del x, dy, xd, y, dx, dg, ws
    torch.cuda.empty_cache()
    epilogue = {}
    for name, thr in (("c3", None), ("c4", -10.0)):
        q, k, v, lf, _, _ = synth(WORKLOADS[name], "cuda")
        gate = g.detach().view(B, T, G, D)
        variants = {
            "attention_fwd_ms": lambda: forgetting_attention(q, k, v, lf, adaptive_threshold=thr),
            "attention_then_norm_ms": lambda: group_norm_gated(
                forgetting_attention(q, k, v, lf, adaptive_threshold=thr).view(B, T, G * D), gate.view(B, T, G * D), wd, None,
                "sigmoid", is_rms_norm=True, num_groups=G),
            "norm_in_epilogue_ms": lambda: forgetting_attention_norm_gate(q, k, v, lf, gate, wd, adaptive_threshold=thr),
        }
        rounds, acc = 4, {key: 0.0 for key in variants}
        with torch.no_grad():   # the variants take turns, so that drifts of the clock hit them alike
            for _ in range(rounds):
                for key, fn in variants.items():
                    acc[key] += event_time(fn, max(5, ns.steps)) * 1e3 / rounds
        epilogue[name if thr is None else f"{name}_threshold_{thr}"] = acc
        del q, k, v, lf
    line = {
        "metric": "gated per-head RMS norm fwd+bwd, algorithmic HBM GB/s (operator incl. autograd)",
        "value": (bytes_f + bytes_b) / sec * 1e-9, "unit": "GB/s", "n_gpus": 1, "steps": ns.steps, "warmup": ns.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"norm_gate: B{B} T{T} heads{G} D{D} bf16 fwd+bwd, sigmoid gate, fp32 weight"},
        "roofline": {"kernel": "norm_gate_bwd", "bound": "hbm", "achieved": kernels["norm_gate_bwd"]["gbps"],
                     "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": kernels["norm_gate_bwd"]["gbps"] / PEAK_HBM_GBPS,
                     "traffic": None, "algorithmic_bytes": bytes_b,
                     "avg_launch_ms": t_b * 1e3},
        "kernels": kernels,
        "attention_epilogue": epilogue,
    }
    print(json.dumps(line))


def power_report(ns):
    """--workload power: socket power and shader clock beside every MFMA kernel of config 3 (or of `--power-of`).

    A child process samples the SMI library every 20 ms while this process runs, one after the other and for at least
    `--seconds` each: nothing (idle), the forward, the dQ kernel and the dK/dV kernel of config 3 alone, the three on
    all-zero q, k, v, dO (same instruction stream, no data toggling), a loop of register-resident MFMAs and a bf16 GEMM of
    the vendor library (8192^3), each on N(0,1) and on all-zero operands, for scale.  Per phase: average launch time, TFLOP/s of executed matmuls, and mean / max power and mean
    clock over the samples of the phase (its first 0.5 s dropped)."""
    import subprocess
    import tempfile
    from forgetting_transformer.ops import _lib
    from forgetting_transformer.ops.forgetting_attention import _view

    tmp = tempfile.mkdtemp(prefix="fox_power_")
    csv_path, stop_path = os.path.join(tmp, "samples.csv"), os.path.join(tmp, "stop")
    child = subprocess.Popen([sys.executable, str(Path(__file__).resolve()), "--power-sampler", csv_path, stop_path])
    try:
        lib = _lib.load()
        w = WORKLOADS[ns.power_of]
        unit = flops_fwd(w) / 2.0
        phases = []

        def run_phase(name, fn, flops):
            t_launch = event_time(fn, 5) if fn else 0.0
            n = max(1, int(ns.seconds / max(t_launch, 1e-4)))
            torch.cuda.synchronize()
            t0 = time.time()
            if fn is None:
                time.sleep(ns.seconds)
                sec = 0.0
            else:
                sec = event_time(fn, n, warmup=0)
            torch.cuda.synchronize()
            phases.append({"phase": name, "t0": t0, "t1": time.time(), "ms_per_launch": sec * 1e3, "launches": n,
                           "tflops": flops / sec * 1e-12 if sec else 0.0})

        run_phase("idle", None, 0.0)
        for zero in (False, True):
            tensors = synth(w, "cuda")
            if zero:
                tensors = tuple(torch.zeros_like(t) if i in (0, 1, 2, 4) else t for i, t in enumerate(tensors))
            q, k, v, log_fgate, dout, _ = tensors
            q, k, v, dout = (x.transpose(1, 2) for x in (q, k, v, dout))
            log_fgate = log_fgate.transpose(1, 2)
            B, H, M, D = q.shape
            N = k.shape[2]
            stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            dims = _lib.Dims(B, H, M, N, D, _lib.DTYPE_BF16)
            c, lse = (torch.empty((B, H, n_), dtype=torch.float32, device="cuda") for n_ in (N, M))
            o, dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
            delta, drow, dc, dg = (torch.empty((B, H, n_), dtype=torch.float32, device="cuda") for n_ in (M, M, N, N))
            fwd = _lib.FwdArgs(dims, _view(q), _view(k), _view(v), _view(o), c.data_ptr(), lse.data_ptr(), None, None,
                               1.0 / math.sqrt(D), None, None, 0)
            bwd = _lib.BwdArgs(dims, _view(q), _view(k), _view(v), _view(o), _view(dout), _view(dq), _view(dk), _view(dv),
                               c.data_ptr(), lse.data_ptr(), None, None, 1.0 / math.sqrt(D), delta.data_ptr(), drow.data_ptr(),
                               dc.data_ptr(), dg.data_ptr(), 0, 0, 0, None, None)
            _lib.check(lib.fox_cumsum_fwd(log_fgate.data_ptr(), *log_fgate.stride(), None, c.data_ptr(), B, H, N, stream), "scan")
            tag = " (all-zero q, k, v, dO)" if zero else ""
            run_phase("fwd" + tag, lambda: _lib.check(lib.fox_attn_fwd(C.byref(fwd), stream), "fwd"), 2 * unit)
            run_phase("bwd_dq" + tag, lambda: _lib.check(lib.fox_attn_bwd_dq(C.byref(bwd), stream), "dq"), 3 * unit)
            run_phase("bwd_dkdv" + tag, lambda: _lib.check(lib.fox_attn_bwd_dkdv(C.byref(bwd), stream), "dkdv"), 4 * unit)
            del tensors, q, k, v, dout, o, dq, dk, dv
            torch.cuda.empty_cache()
        # a loop of nothing but register-resident MFMAs (fox_probe_mfma): what the power limit leaves of the matrix peak
        n_cu = torch.cuda.get_device_properties(0).multi_processor_count
        sink = torch.zeros(1, device="cuda", dtype=torch.float32)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        probe_iters = 20000
        for zero in (False, True):
            operands = torch.zeros(16 * 64 * 8, device="cuda", dtype=torch.bfloat16)
            if not zero:
                operands.normal_()
            run_phase("MFMA loop, operands in registers" + (" (all-zero operands)" if zero else ""),
                      lambda: _lib.check(lib.fox_probe_mfma(operands.data_ptr(), sink.data_ptr(), n_cu, probe_iters, stream), "probe"),
                      n_cu * 4 * probe_iters * 32 * 32768.0)
        for zero in (False, True):
            a = torch.zeros(8192, 8192, device="cuda", dtype=torch.bfloat16)
            b = torch.zeros(8192, 8192, device="cuda", dtype=torch.bfloat16)
            if not zero:
                a.normal_()
                b.normal_()
            out = torch.empty_like(a)
            run_phase("vendor GEMM 8192^3 bf16" + (" (all-zero operands)" if zero else ""),
                      lambda: torch.matmul(a, b, out=out), 2.0 * 8192 ** 3)
    finally:
        open(stop_path, "w").close()
        child.wait(timeout=30)
    header, samples = [], []
    for ln in open(csv_path):
        if ln.startswith("#"):
            header.append(ln[2:].strip())
        elif ln[0].isdigit():
            f = ln.strip().split(",")
            samples.append((float(f[0]), float(f[1]), float(f[2]), float(f[3]), float(f[4]), f[5]))
    for ph in phases:
        sel = [x for x in samples if ph["t0"] + 0.5 <= x[0] <= ph["t1"]]
        ph["samples"] = len(sel)
        if sel:
            ph["socket_w_mean"] = sum(x[1] for x in sel) / len(sel)
            ph["socket_w_max"] = max(x[1] for x in sel)
            ph["gfx_mhz_mean"] = sum(x[2] for x in sel) / len(sel)
            ph["gfx_mhz_max_xcd_mean"] = sum(x[3] for x in sel) / len(sel)
            ph["hotspot_c_max"] = max(x[4] for x in sel)
            ph["throttle_status"] = sorted({x[5] for x in sel})
        ph["frac_of_bf16_peak"] = ph["tflops"] / PEAK_BF16_TFLOPS
        del ph["t0"], ph["t1"]
    span = samples[-1][0] - samples[0][0] if len(samples) > 1 else 0.0
    dk = next(p for p in phases if p["phase"] == "bwd_dkdv")
    print(json.dumps({
        "metric": f"socket power and shader clock beside the MFMA kernels of B{w['B']} T{w['M']} H{w['H']} D{w['D']} bf16", "value": dk.get("socket_w_mean"),
        "unit": "W (dK/dV kernel)", "n_gpus": 1, "higher_is_better": False, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"power: {ns.power_of} kernels one at a time, {ns.seconds:g} s each, SMI sampled every 20 ms"},
        "sampler": {"samples": len(samples), "rate_hz": len(samples) / span if span else 0.0, "notes": header},
        "phases": phases}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS) + ["shift", "norm_gate", "ref_sweep", "acp_sweep", "power"])
    ap.add_argument("--seconds", type=float, default=3.0, help="--workload power: duration of every phase")
    ap.add_argument("--power-of", default="c3", choices=["c3", "c3d64", "c3d32", "c3d16"],
                    help="--workload power: the workload whose kernels run")
    ap.add_argument("--threshold", default=None,
                    help="adaptive_threshold of the main workload: a float or 'auto' (default: no pruning); with it the "
                         "roofline entry prices the dK/dV pass against HBM, the bound of a heavily pruned step")
    ap.add_argument("--no-extras", action="store_true", help="skip the ACP and chunked-prefill reports")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy three times (a kernel of known traffic to scale HBM counters by)")
    ns = ap.parse_args()
    if ns.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: Forgetting Attention never communicates (every (batch, head) pair is an "
                 "independent problem), so a multi-GPU run would only replicate this measurement. Use --gpus 1.")
    if ns.workload == "power":   # starts its sampler process before this process touches the GPU
        return power_report(ns)
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an AMD GPU (there is no CPU path for the operator)")

    from forgetting_transformer import forgetting_attention

    if ns.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if ns.workload == "shift":
        return shift_report(ns)
    if ns.workload == "norm_gate":
        return norm_gate_report(ns)
    if ns.workload == "acp_sweep":
        return acp_sweep_report(ns)
    if ns.workload == "ref_sweep":
        return ref_sweep_report(ns)

    w = WORKLOADS[ns.workload]
    tensors = synth(w, "cuda")
    q, k, v, log_fgate, dout, seq_start = tensors
    if not w["fwd_only"]:
        q, k, v, log_fgate = (x.requires_grad_() for x in (q, k, v, log_fgate))
    thr = None if ns.threshold is None else ("auto" if ns.threshold == "auto" else float(ns.threshold))

    def step():
        if w["fwd_only"]:
            with torch.no_grad():
                forgetting_attention(q, k, v, log_fgate, head_first=w["head_first"], seq_start=seq_start, adaptive_threshold=thr)
        else:
            out = forgetting_attention(q, k, v, log_fgate, head_first=w["head_first"], seq_start=seq_start,
                                       adaptive_threshold=thr)
            out.backward(dout)
            q.grad = k.grad = v.grad = log_fgate.grad = None

    sec = time_steps(step, ns.steps, ns.warmup)
    f_fwd = flops_fwd(w)
    total = f_fwd if w["fwd_only"] else 3.5 * f_fwd  # bwd = 2.5 x fwd in the reference's convention
    value = total / sec * 1e-12

    stage_thr = thr
    if thr == "auto":   # the (batch, head) thresholds the operator would derive, from the library's own kernel
        from forgetting_transformer.ops import _lib
        from forgetting_transformer.ops.forgetting_attention import _view
        qh, kh = (x.detach().transpose(1, 2) if not w["head_first"] else x.detach() for x in (q, k))
        stage_thr = torch.empty((w["B"], w["H"]), dtype=torch.float32, device="cuda")
        scratch = torch.empty((w["B"], w["H"], 3), dtype=torch.int32, device="cuda")
        dims = _lib.Dims(w["B"], w["H"], w["M"], w["N"], w["D"], _lib.DTYPE_BF16)
        qv, kv = _view(qh), _view(kh)
        _lib.check(_lib.load().fox_auto_threshold(C.byref(dims), C.byref(qv), C.byref(kv), 1.0 / math.sqrt(w["D"]),
                                                  stage_thr.data_ptr(), scratch.data_ptr(),
                                                  C.c_void_p(torch.cuda.current_stream().cuda_stream)), "fox_auto_threshold")
    stages = stage_times(w, tensors, max(3, ns.steps), threshold=stage_thr)
    unit_flops = f_fwd / 2.0  # one causal matmul, B*H*T^2*D
    kern_flops = {"fwd": 2 * unit_flops, "bwd_dkdv": 4 * unit_flops, "bwd_dq": 3 * unit_flops}
    kernels = {}
    for name, t in stages.items():
        e = {"ms": t * 1e3}
        if name in kern_flops:
            e["tflops"] = kern_flops[name] / t * 1e-12
            e["frac_of_peak"] = e["tflops"] / PEAK_BF16_TFLOPS
        kernels[name] = e
    traffic, traffic_source = measured_traffic(ns.workload if thr is None else ns.workload + "_pruned")
    if w["fwd_only"]:  # few query rows against a long key sequence: one pass over K and V, HBM-bound
        dom = "fwd"
        pad = seq_start.float() if seq_start is not None else torch.zeros(w["B"], device="cuda")
        alg_bytes = ((2.0 * w["H"] * (w["N"] - pad) * w["D"] * 2).sum().item()
                     + 2 * w["B"] * w["H"] * w["M"] * w["D"] * 2 + w["B"] * w["H"] * w["N"] * 4)
        gbps = alg_bytes / stages[dom] * 1e-9
        roofline = {"kernel": dom, "bound": "hbm", "achieved": gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                    "frac": gbps / PEAK_HBM_GBPS, "traffic": traffic, "traffic_source": traffic_source,
                    "algorithmic_bytes": alg_bytes, "avg_launch_ms": kernels[dom]["ms"]}
    elif thr is not None:   # pruned step: every kernel is a stream over its inputs and outputs; dK/dV is the longest
        dom = "bwd_dkdv"
        S_, R_ = w["B"] * w["H"] * w["M"] * w["D"] * 2, w["B"] * w["H"] * w["M"] * 4
        alg_bytes = 6 * S_ + 6 * R_   # q, k, v, do in; dk, dv out; lse, delta, row sums, c (rows and keys) in, dc out
        gbps = alg_bytes / stages[dom] * 1e-9
        roofline = {"kernel": dom, "bound": "hbm", "achieved": gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                    "frac": gbps / PEAK_HBM_GBPS, "traffic": traffic, "traffic_source": traffic_source,
                    "algorithmic_bytes": alg_bytes, "avg_launch_ms": kernels[dom]["ms"]}
    else:
        dom = "bwd_dkdv"
        roofline = {"kernel": dom, "bound": "mfma", "achieved": kernels[dom]["tflops"], "peak": PEAK_BF16_TFLOPS,
                    "unit": "TFLOP/s", "frac": kernels[dom]["tflops"] / PEAK_BF16_TFLOPS, "traffic": traffic,
                    "traffic_source": traffic_source, "algorithmic_flops": kern_flops[dom],
                    "avg_launch_ms": kernels[dom]["ms"]}

    line = {
        "metric": "fwd+bwd TFLOP/s & % bf16 MFMA peak, T=16k D=128; ACP speedup vs no-prune",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": ns.steps, "warmup": ns.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{ns.workload}: B{w['B']} M{w['M']} N{w['N']} H{w['H']} D{w['D']} bf16 "
                               f"{'fwd' if w['fwd_only'] else 'fwd+bwd'}, gate logits N({w['mean']},{w['std']}), "
                               f"head_first={w['head_first']}, "
                               + ("no pruning" if thr is None else f"adaptive_threshold={thr}"),
                   "flops_convention": "fwd 2*B*H*T^2*D, bwd 5*B*H*T^2*D (causal)"},
        "frac_of_bf16_peak": value / PEAK_BF16_TFLOPS,
        "roofline": roofline,
        "kernels": kernels,
    }
    if not w["fwd_only"] and thr is None:
        # the convention credits the backward 5 x B*H*T^2*D; its two kernels execute 3 + 4 (S and dP are recomputed in both)
        bwd_s = stages["bwd_dq"] + stages["bwd_dkdv"]
        line["backward_credited_frac"] = 5 * unit_flops / bwd_s * 1e-12 / PEAK_BF16_TFLOPS
        line["backward_executed_frac"] = 7 * unit_flops / bwd_s * 1e-12 / PEAK_BF16_TFLOPS
    if not ns.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
    if not ns.no_extras and ns.workload == "c3":
        del q, k, v, log_fgate, dout, tensors
        torch.cuda.empty_cache()
        line["acp"] = acp_report(max(2, ns.steps // 2), 1)
        torch.cuda.empty_cache()
        line["prefill"] = prefill_report(max(5, ns.steps), 2)
        torch.cuda.empty_cache()
        line["decode"] = decode_report(max(5, ns.steps), 2)
        torch.cuda.empty_cache()
        line["head_dim_64"] = head_dim_report(max(2, ns.steps // 2), 1)
        for name in ("c3d32", "c3d16"):
            torch.cuda.empty_cache()
            line["head_dim_" + name[3:]] = head_dim_report(max(2, ns.steps // 2), 1, name)
        torch.cuda.empty_cache()
        line["library_example"] = small_shape_report(ns.steps, ns.warmup)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
