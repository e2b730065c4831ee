"""Writes the committed golden vectors under tests/golden/.

The reference holds no fixtures for Forgetting Attention (its only test builds its
inputs on a CUDA device at run time), so these vectors come from this repository's
own oracle, whose functions are pinned in tests/test_oracle_cpu.py.  Inputs follow
Benchmark configuration 1: B=2, T=256, H=4, D=64, q/k/v ~ N(0,1), log_fgate =
logsigmoid(N(0,1)), sm_scale = 1/8, (batch, time, head, dim) layout, fp32.
A second file holds a small bf16 forward+backward case with left padding and
seqlen_q < seqlen_k, including gradients, for the GPU parity test.

    python tests/golden/make_golden.py
"""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle.fox_oracle import forgetting_attention_ref, forgetting_attention_ref_grads  # noqa: E402

HERE = Path(__file__).resolve().parent


def c1():
    g = torch.Generator().manual_seed(20250101)
    B, T, H, D = 2, 256, 4, 64
    q, k, v = (torch.randn((B, T, H, D), generator=g) for _ in range(3))
    log_fgate = torch.nn.functional.logsigmoid(torch.randn((B, T, H), generator=g))
    out, lse = forgetting_attention_ref(q, k, v, log_fgate, sm_scale=1 / 8, return_lse=True)
    np.savez_compressed(HERE / "c1_b2_t256_h4_d64.npz", q=q.numpy(), k=k.numpy(), v=v.numpy(),
                        log_fgate=log_fgate.numpy(), out=out.numpy(), lse=lse.numpy())


def small_bwd():
    g = torch.Generator().manual_seed(20250102)
    B, H, M, N, D = 2, 2, 72, 200, 32
    q = torch.randn((B, H, M, D), generator=g).bfloat16()
    k = torch.randn((B, H, N, D), generator=g).bfloat16()
    v = torch.randn((B, H, N, D), generator=g).bfloat16()
    log_fgate = torch.nn.functional.logsigmoid(torch.randn((B, H, N), generator=g) + 1.0)
    dout = torch.randn((B, H, M, D), generator=g).bfloat16()
    seq_start = torch.tensor([0, 150], dtype=torch.long)   # second row: queries 0..21 see no key at all
    out, dq, dk, dv, dg = forgetting_attention_ref_grads(q, k, v, log_fgate, dout, head_first=True, seq_start=seq_start,
                                                         sm_scale=0.25, compute_dtype=torch.float64)
    f = lambda x: x.float().numpy()
    np.savez_compressed(HERE / "bwd_b2_h2_m72_n200_d32.npz", q=f(q), k=f(k), v=f(v), log_fgate=log_fgate.numpy(),
                        dout=f(dout), seq_start=seq_start.numpy(), out=f(out), dq=f(dq), dk=f(dk), dv=f(dv), dlog_fgate=f(dg))


if __name__ == "__main__":
    c1()
    small_bwd()
    for p in sorted(HERE.glob("*.npz")):
        print(p.name, p.stat().st_size)
