"""Shared fixtures: import paths, the ``gpu`` marker, seeded synthetic inputs."""
import math
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
for p in (ROOT / "forgetting-transformer_amd", ROOT):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real AMD GPU (run on the MI355X box)")


def make_inputs(B, H, M, N, D, *, dtype=torch.bfloat16, device="cpu", seed=0, gate_mean=0.0, gate_std=1.0,
                gate_uniform=None, qkv_std=1.0, head_first=True, seq_start=None, requires_grad=False):
    """Seeded synthetic inputs in the distributions the benchmark configurations name.

    Everything is drawn on the CPU in fp32 (so CPU and GPU runs see the same values)
    and then cast / moved.  Returns q, k, v, log_fgate, dout (+ seq_start tensor).
    """
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, M, D), generator=g) * qkv_std
    k = torch.randn((B, H, N, D), generator=g) * qkv_std
    v = torch.randn((B, H, N, D), generator=g) * qkv_std
    if gate_uniform is not None:
        logits = torch.rand((B, H, N), generator=g) * (gate_uniform[1] - gate_uniform[0]) + gate_uniform[0]
    else:
        logits = torch.randn((B, H, N), generator=g) * gate_std + gate_mean
    log_fgate = torch.nn.functional.logsigmoid(logits)
    dout = torch.randn((B, H, M, D), generator=g)
    ss = None
    if seq_start == "random":
        ss = torch.randint(0, N, (B,), generator=g, dtype=torch.long)
    elif seq_start is not None:
        ss = torch.as_tensor(seq_start, dtype=torch.long)
    q, k, v, dout = (x.to(dtype) for x in (q, k, v, dout))
    if dtype == torch.float64:
        log_fgate = log_fgate.double()
    if not head_first:
        q, k, v, dout = (x.transpose(1, 2).contiguous() for x in (q, k, v, dout))
        log_fgate = log_fgate.transpose(1, 2).contiguous()
    q, k, v, log_fgate, dout = (x.to(device) for x in (q, k, v, log_fgate, dout))
    if ss is not None:
        ss = ss.to(device)
    if requires_grad:
        for x in (q, k, v, log_fgate):
            x.requires_grad_()
    return q, k, v, log_fgate, dout, ss
