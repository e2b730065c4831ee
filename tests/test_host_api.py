"""Host-side contract of the operator, checked without a GPU: the shared library
loads and exports every symbol the public header declares, argument validation in
the C ABI returns error codes before anything is launched, and the Python wrapper
raises the reference's error types (ops/forgetting_attention.py:78-137, 447-448)."""
import ctypes as C
import math
import re

import pytest
import torch

from conftest import ROOT
from forgetting_transformer import forgetting_attention
from forgetting_transformer.ops import _lib
from forgetting_transformer.ops.forgetting_attention import ForgettingAttention, maybe_contiguous


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "fox_attn.h").read_text()
    declared = set(re.findall(r"^\s*(?:int|int32_t|int64_t|const char\*)\s+(fox_\w+)\s*\(", header, flags=re.M))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.fox_version() >= 100


def test_public_header_is_plain_c(tmp_path):
    """include/fox_attn.h must be usable from C and from C++ as it stands (the boundary is a C ABI): it compiles,
    warning-free, as C99 and as C++11, and a C program that uses it links against the library and runs its host-only
    calls (no device needed: version, tile table, an argument check that fails before any launch)."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no host C compiler")
    src = tmp_path / "use_header.c"
    src.write_text(f"""
#include <stdio.h>
#include <string.h>
#include "{ROOT / 'include' / 'fox_attn.h'}"
int main(void) {{
  int32_t bm = 0, bn = 0, kn = 0, km = 0;
  fox_fwd_args args;
  memset(&args, 0, sizeof args);
  if (fox_version() < 100) return 1;
  if (fox_tile_config(128, &bm, &bn, &kn, &km) != FOX_OK || bm <= 0 || bn <= 0) return 2;
  if (fox_tile_config(48, &bm, &bn, &kn, &km) == FOX_OK) return 3;
  if (fox_attn_fwd(&args, NULL) == FOX_OK) return 4;      /* all-zero dims: rejected on the host */
  if (strlen(fox_last_error()) == 0) return 5;
  printf("%d %d\\n", bm, bn);
  return 0;
}}
""")
    for cmd in (["gcc", "-std=c99"], ["g++", "-std=c++11", "-x", "c++"]):
        subprocess.run(cmd + ["-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", str(src)], check=True)
    exe = tmp_path / "use_header"
    lib_dir = _lib.LIB_PATH.parent
    subprocess.run(["gcc", "-std=c99", str(src), "-o", str(exe), f"-L{lib_dir}", "-lfox_attn", f"-Wl,-rpath,{lib_dir}"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert [int(x) for x in out] == list(_lib.tile_config(128)[:2])


def test_kernels_do_not_spill():
    """The compiler's resource report, written next to the library by the build: the MFMA kernels must
    keep every register in the register file (a spill multiplies their run time) at the occupancy
    they are designed for, and must fit the 160 KiB of LDS of a CU at that occupancy."""
    import json
    path = _lib.LIB_PATH.with_name("kernel_resources.json")
    assert path.exists(), f"{path} is missing: rebuild with python forgetting-transformer_amd/build.py --force"
    usage = json.loads(path.read_text())
    want = {"fwd_kernel": 2, "dq_kernel": 2, "dkdv_kernel": 1}          # waves per SIMD
    seen = set()
    for name, u in usage.items():
        for kernel, occupancy in want.items():
            if f"fox{len(kernel)}{kernel}I" in name.replace("_ZN3", ""):
                seen.add(kernel)
                assert u["ScratchSize"] == 0 and u["VGPRs Spill"] == 0, (name, u)
                assert u["Occupancy"] >= occupancy, (name, u)
                assert u["LDS Size"] * occupancy <= 160 * 1024, (name, u)
    assert seen == set(want)
    for name, u in usage.items():                                        # nothing else spills either
        assert u["ScratchSize"] == 0, (name, u)


def test_tile_config():
    for d in (16, 32, 64, 128):
        bm, bn, kbn, kbm = _lib.tile_config(d)
        assert bm % 32 == 0 and bn % 32 == 0 and kbn % 32 == 0 and kbm % 32 == 0
    with pytest.raises(RuntimeError, match="head dim"):
        _lib.tile_config(48)


def test_c_abi_rejects_bad_arguments_before_launching():
    lib = _lib.load()
    buf = (C.c_char * 4096)()
    base = C.addressof(buf)
    base += (-base) % 16
    view = _lib.View(base, 64, 64, 64)

    def fwd(dims, q=view, log_lambda=base):
        a = _lib.FwdArgs(dims, q, view, view, view, log_lambda, base, None, None, 1.0, None)
        return lib.fox_attn_fwd(C.byref(a), None)

    assert fwd(_lib.Dims(1, 1, 8, 8, 48, 0)) == -1 and b"head dim" in lib.fox_last_error()
    assert fwd(_lib.Dims(1, 1, 9, 8, 64, 0)) == -1 and b"M=9 > N=8" in lib.fox_last_error()
    assert fwd(_lib.Dims(0, 1, 8, 8, 64, 0)) == -1
    assert fwd(_lib.Dims(1, 1, 8, 8, 64, 7)) == -1 and b"dtype" in lib.fox_last_error()
    assert fwd(_lib.Dims(1, 1, 8, 8, 64, 0), q=_lib.View(None, 64, 64, 64)) == -1 and b"q is NULL" in lib.fox_last_error()
    assert fwd(_lib.Dims(1, 1, 8, 8, 64, 0), q=_lib.View(base + 2, 64, 64, 64)) == -2
    assert fwd(_lib.Dims(1, 1, 8, 8, 64, 0), q=_lib.View(base, 64, 64, 12)) == -2 and b"strides" in lib.fox_last_error()
    assert fwd(_lib.Dims(1, 1, 8, 8, 64, 0), log_lambda=None) == -1
    assert lib.fox_attn_fwd(None, None) == -1
    assert lib.fox_attn_bwd(None, None) == -1
    assert lib.fox_cumsum_fwd(None, 1, 1, 1, None, base, 1, 1, 8, None) == -1
    assert lib.fox_cumsum_bwd(base, base, 0, 0, 0, None, 1, 1, 8, None) == -1 and b"alias" in lib.fox_last_error()
    assert lib.fox_gate_cumsum_fwd(None, 0, 1, 1, 1, None, None, base, 1, 1, 8, None) == -1
    assert lib.fox_gate_cumsum_fwd(base, 3, 1, 1, 1, None, None, base + 64, 1, 1, 8, None) == -1 and b"logits_dtype" in lib.fox_last_error()
    assert lib.fox_gate_cumsum_bwd(base, base + 64, 0, 1, 1, 1, None, base + 64, 1, 1, 1, 1, 1, 8, None) == -1 and b"alias" in lib.fox_last_error()
    assert lib.fox_gate_cumsum_bwd(base, base + 64, 0, 1, 1, 1, None, None, 1, 1, 1, 1, 1, 8, None) == -1
    assert lib.fox_probe_mfma(None, base, 1, 1, None) == -1 and b"fox_probe_mfma" in lib.fox_last_error()
    assert lib.fox_probe_mfma(base, base, 0, 1, None) == -1 and lib.fox_probe_mfma(base, base, 1, 0, None) == -1
    with pytest.raises(RuntimeError, match="code -1"):
        _lib.check(-1, "x")


def test_token_shift_c_abi_and_wrapper_checks():
    lib = _lib.load()
    buf = (C.c_char * 4096)()
    base = C.addressof(buf)
    base += (-base) % 16

    def args(D=64, dtype=0, x=base, out=base + 1024, xs=(512, 64, 64), dout=None, dx=None, dprev=None, dcurr=None):
        return _lib.ShiftArgs(1, 2, 1, D, dtype, x, *xs, base + 2048, base + 2304, 2, 1, 1, out, dout, dx, dprev, dcurr)

    assert lib.fox_token_shift_fwd(C.byref(args(D=48)), None) == -1 and b"head dim" in lib.fox_last_error()
    assert lib.fox_token_shift_fwd(C.byref(args(dtype=3)), None) == -1 and b"dtype" in lib.fox_last_error()
    assert lib.fox_token_shift_fwd(C.byref(args(x=None)), None) == -1
    assert lib.fox_token_shift_fwd(C.byref(args(out=None)), None) == -1 and b"out" in lib.fox_last_error()
    assert lib.fox_token_shift_fwd(C.byref(args(out=base)), None) == -1 and b"alias" in lib.fox_last_error()
    assert lib.fox_token_shift_fwd(C.byref(args(x=base + 2)), None) == -2
    assert lib.fox_token_shift_fwd(C.byref(args(xs=(512, 60, 64))), None) == -2 and b"strides" in lib.fox_last_error()
    assert lib.fox_token_shift_bwd(C.byref(args()), None) == -1            # dout, dx missing
    assert lib.fox_token_shift_bwd(C.byref(args(dout=base + 1024, dx=base + 1024, dprev=base, dcurr=base)), None) == -1
    assert lib.fox_token_shift_fwd(None, None) == -1 and lib.fox_token_shift_bwd(None, None) == -1

    from forgetting_transformer import token_shift
    x = torch.randn(2, 8, 2, 64).bfloat16()
    w = torch.rand(2, 8, 2)
    with pytest.raises(AssertionError):
        token_shift(torch.randn(2, 8, 2, 48).bfloat16(), w, w)            # head dim (token_shift.py:164)
    with pytest.raises(AssertionError):
        token_shift(x, w[:, :4], w)                                        # weight shape (:165)
    with pytest.raises(AssertionError):
        token_shift(x, w.transpose(0, 1).contiguous().transpose(0, 1), w)  # weight strides differ (:166)
    with pytest.raises(AssertionError):
        token_shift(x.float(), w, w)
    with pytest.raises(RuntimeError, match="no CPU path"):
        token_shift(x, w, w)


def test_norm_gate_c_abi_and_wrapper_checks():
    lib = _lib.load()
    buf = (C.c_char * 8192)()
    base = C.addressof(buf)
    base += (-base) % 16

    def args(D=64, dtype=0, act=0, x=base, y=base + 1024, xs=64, rstd=base + 4096, weight=base + 2048, g=base + 512):
        return _lib.NormGateArgs(2, 1, D, dtype, act, 1e-6, x, xs, g, 64, weight, y, 64, rstd,
                                 None, 0, None, 0, None, 0, None, None)

    assert lib.fox_norm_gate_fwd(C.byref(args(D=48)), None) == -1 and b"head dim" in lib.fox_last_error()
    assert lib.fox_norm_gate_fwd(C.byref(args(dtype=2)), None) == -1 and b"dtype" in lib.fox_last_error()
    assert lib.fox_norm_gate_fwd(C.byref(args(act=5)), None) == -1 and b"activation" in lib.fox_last_error()
    assert lib.fox_norm_gate_fwd(C.byref(args(x=None)), None) == -1
    assert lib.fox_norm_gate_fwd(C.byref(args(g=None)), None) == -1 and b"g must not be NULL" in lib.fox_last_error()
    # the plain norm (FOX_ACT_NONE) takes no gate, and is checked like the gated one otherwise
    assert lib.fox_norm_gate_fwd(C.byref(args(act=2, g=None, y=None)), None) == -1 and b"y must not be NULL" in lib.fox_last_error()
    assert lib.fox_norm_gate_fwd(C.byref(args(act=2, g=None, xs=60)), None) == -2
    assert lib.fox_norm_gate_bwd(C.byref(args(act=2, g=None)), None) == -1      # dy, dx missing
    assert lib.fox_norm_gate_fwd(C.byref(args(y=None)), None) == -1 and b"y must not be NULL" in lib.fox_last_error()
    assert lib.fox_norm_gate_fwd(C.byref(args(x=base + 4)), None) == -2
    assert lib.fox_norm_gate_fwd(C.byref(args(xs=60)), None) == -2 and b"row strides" in lib.fox_last_error()
    assert lib.fox_norm_gate_bwd(C.byref(args()), None) == -1        # dy, dx, dg missing
    assert lib.fox_norm_gate_fwd(None, None) == -1 and lib.fox_norm_gate_bwd(None, None) == -1
    nb = C.c_int64(0)
    assert lib.fox_norm_gate_workspace_bytes(65536, 16, 128, C.byref(nb)) == 0
    assert nb.value == (2048 + 64) * 16 * 128 * 4                     # one row per 32-row strip + one per 32 strips
    assert lib.fox_norm_gate_workspace_bytes(1, 1, 48, C.byref(nb)) == -1
    assert lib.fox_norm_gate_workspace_bytes(1, 1, 64, None) == -1

    from forgetting_transformer import group_norm_gated
    x = torch.randn(4, 128).bfloat16()
    w = torch.ones(128)
    with pytest.raises(NotImplementedError):
        group_norm_gated(x, x, w, torch.zeros(128), "sigmoid", is_rms_norm=True, num_groups=2)
    with pytest.raises(NotImplementedError):
        group_norm_gated(x, x, w, None, "sigmoid", residual=x, is_rms_norm=True, num_groups=2)
    with pytest.raises(ValueError):
        group_norm_gated(x, x, w, None, "tanh", is_rms_norm=True, num_groups=2)
    with pytest.raises(ValueError, match="divisible"):
        group_norm_gated(x, x, w, None, "sigmoid", is_rms_norm=True, num_groups=3)
    with pytest.raises(AssertionError):
        group_norm_gated(x.float(), x.float(), w, None, "sigmoid", is_rms_norm=True, num_groups=2)
    with pytest.raises(RuntimeError, match="no CPU path"):
        group_norm_gated(x, x, w, None, "sigmoid", is_rms_norm=True, num_groups=2)

    from forgetting_transformer import group_norm, rms_norm
    with pytest.raises(NotImplementedError):
        group_norm(x, w, torch.zeros(128), is_rms_norm=True, num_groups=2)     # bias
    with pytest.raises(NotImplementedError):
        group_norm(x, w, None, is_rms_norm=False, num_groups=2)                # mean-centred norm
    with pytest.raises(ValueError, match="divisible"):
        group_norm(x, w, None, is_rms_norm=True, num_groups=3)                 # layernorm.py:723-724
    with pytest.raises(AssertionError):
        group_norm(x.float(), w, None, is_rms_norm=True, num_groups=2)
    with pytest.raises(RuntimeError, match="no CPU path"):
        rms_norm(x, w)


def test_qk_norm_threshold_matches_the_layer_rule():
    """modeling_forgetting_transformer.py:371-380, both weight-sharing modes."""
    from forgetting_transformer import qk_norm_threshold
    H, D, T, tol = 3, 16, 777, -12.0
    gen = torch.Generator().manual_seed(3)
    wq, wk = torch.randn(H * D, generator=gen), torch.randn(H * D, generator=gen)
    thr = qk_norm_threshold(wq, wk, H, D, T, tol)
    assert thr.shape == (H,) and thr.dtype == torch.float32 and not thr.requires_grad
    for h in range(H):
        want = -(2 * wq[h * D:(h + 1) * D].abs().max() * wk[h * D:(h + 1) * D].abs().max() * math.sqrt(D) + math.log(T)) + tol
        assert torch.allclose(thr[h], want, rtol=1e-6)
    thr0 = qk_norm_threshold(wq[:D], wk[:D], H, D, T, tol, share_param_across_head=True)
    assert thr0.shape == () and torch.allclose(thr0, thr[0], rtol=1e-6)
    with pytest.raises(AssertionError):
        qk_norm_threshold(wq[:D], wk[:D], H, D, T, tol)                        # per-head weights expected (:376)


def test_workspace_query():
    lib = _lib.load()
    need = C.c_int64(-1)
    assert lib.fox_attn_fwd_workspace_bytes(C.byref(_lib.Dims(4, 16, 16384, 16384, 128, 0)), C.byref(need)) == 0
    assert need.value == 0                          # plenty of query tiles: never split
    assert lib.fox_attn_fwd_workspace_bytes(C.byref(_lib.Dims(16, 16, 128, 32768, 128, 0)), C.byref(need)) == 0
    assert need.value > 0 and need.value % (16 * 16 * 128 * 130 * 4) == 0   # splits x rows x (D + 2) floats
    assert lib.fox_attn_fwd_workspace_bytes(C.byref(_lib.Dims(1, 1, 1, 100, 64, 0)), C.byref(need)) == 0 and need.value == 0
    # one query row against a long cache: the streaming kernel takes 2048 / (B*H) splits of at least 512 keys
    assert lib.fox_attn_fwd_workspace_bytes(C.byref(_lib.Dims(16, 16, 1, 32768, 128, 0)), C.byref(need)) == 0
    assert need.value == 8 * 16 * 16 * 130 * 4
    assert lib.fox_attn_fwd_workspace_bytes(C.byref(_lib.Dims(1, 2, 1, 2048, 64, 0)), C.byref(need)) == 0
    assert need.value == 4 * 1 * 2 * 66 * 4
    assert lib.fox_attn_fwd_workspace_bytes(C.byref(_lib.Dims(1, 1, 1, 100, 48, 0)), C.byref(need)) == -1
    assert lib.fox_attn_fwd_workspace_bytes(C.byref(_lib.Dims(1, 1, 1, 100, 64, 0)), None) == -1


def _cpu_inputs(B=2, T=8, H=2, D=64, dtype=torch.bfloat16):
    q = torch.randn(B, T, H, D).to(dtype)
    g = torch.nn.functional.logsigmoid(torch.randn(B, T, H))
    return q, q.clone(), q.clone(), g


def test_wrapper_error_contract():
    q, k, v, g = _cpu_inputs()
    with pytest.raises(AssertionError, match="Only torch.float16 or torch.bfloat16"):
        forgetting_attention(q.float(), k, v, g)
    with pytest.raises(AssertionError, match="head dims"):
        forgetting_attention(q[..., :48], k[..., :48], v[..., :48], g)
    with pytest.raises(AssertionError, match="float32"):
        forgetting_attention(q, k, v, g.bfloat16())
    with pytest.raises(AssertionError):
        forgetting_attention(q, k, v, g[:, :-1])                       # wrong log_fgate shape
    with pytest.raises(AssertionError, match="longer than the query"):
        forgetting_attention(q, k[:, :4], v[:, :4], g[:, :4])          # M > N
    with pytest.raises(AssertionError, match='"auto"'):
        forgetting_attention(q, k, v, g, adaptive_threshold="automatic")
    with pytest.raises(RuntimeError, match="broadcastable"):
        forgetting_attention(q, k, v, g, adaptive_threshold=torch.zeros(3))
    with pytest.raises(AssertionError):
        forgetting_attention(q, k, v, g, seq_start=torch.zeros(5, dtype=torch.long))
    with pytest.raises(AssertionError, match="feature size"):
        forgetting_attention(q, k, v[..., :32], g)


def test_no_cpu_fallback():
    q, k, v, g = _cpu_inputs()
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        forgetting_attention(q, k, v, g)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        forgetting_attention(q, k, v, g, head_first=True, adaptive_threshold=-10.0, seq_start=torch.zeros(2, dtype=torch.long))


def test_norm_gate_epilogue_wrapper_checks():
    """forgetting_attention_norm_gate validates on the host before any launch, has no CPU path, and the C entry point
    rejects a bad epilogue without touching the device."""
    from forgetting_transformer import forgetting_attention_norm_gate
    q, k, v, g = _cpu_inputs()
    B, T, H, D = q.shape
    gate, w = torch.zeros_like(q), torch.ones(H * D)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        forgetting_attention_norm_gate(q, k, v, g, gate, w)
    with pytest.raises(AssertionError, match="weight must have shape"):
        forgetting_attention_norm_gate(q, k, v, g, gate, w[:-1])
    with pytest.raises(AssertionError, match="shape of q"):
        forgetting_attention_norm_gate(q, k, v, g, gate[:, :-1], w)
    with pytest.raises(AssertionError, match="dtype of q"):
        forgetting_attention_norm_gate(q, k, v, g, gate.half() if q.dtype == torch.bfloat16 else gate.bfloat16(), w)
    with pytest.raises(ValueError, match="Unsupported activation"):
        forgetting_attention_norm_gate(q, k, v, g, gate, w, activation="relu")
    with pytest.raises(AssertionError, match="Only torch.float16 or torch.bfloat16"):
        forgetting_attention_norm_gate(q.float(), k, v, g, gate, w)
    lib = _lib.load()
    args, epi = _lib.FwdArgs(), _lib.FwdEpilogue()
    assert lib.fox_attn_fwd_norm_gate(None, C.byref(epi), None) != 0
    assert lib.fox_attn_fwd_norm_gate(C.byref(args), None, None) != 0
    epi.activation = 7
    assert lib.fox_attn_fwd_norm_gate(C.byref(args), C.byref(epi), None) != 0
    assert b"activation" in lib.fox_last_error()
    epi.activation = _lib.ACT_NONE
    assert lib.fox_attn_fwd_norm_gate(C.byref(args), C.byref(epi), None) != 0
    assert b"y is NULL" in lib.fox_last_error()


def test_product_code_never_touches_the_oracle():
    pkg = ROOT / "forgetting-transformer_amd"
    for path in list(pkg.rglob("*.py")) + list(pkg.rglob("*.hip")) + list(pkg.rglob("*.hpp")):
        text = path.read_text()
        assert not re.search(r"\boracle\b", text), path
        assert "_work/" not in text, path


def test_maybe_contiguous_keeps_aligned_views():
    x = torch.zeros(2, 16, 4 * 64, dtype=torch.bfloat16)
    v = x.view(2, 16, 4, 64).transpose(1, 2)        # the (B,H,T,D) view the FoX layer passes (modeling_forgetting_transformer.py:318-320)
    assert maybe_contiguous(v) is v
    odd = torch.zeros(2, 2, 16, 65, dtype=torch.bfloat16)[..., :64]
    assert maybe_contiguous(odd) is not odd and maybe_contiguous(odd).is_contiguous()
    t = torch.zeros(2, 2, 64, 16, dtype=torch.bfloat16).transpose(2, 3)
    assert maybe_contiguous(t).stride(-1) == 1


def test_autograd_function_signature_matches_reference():
    import inspect
    params = list(inspect.signature(ForgettingAttention.forward).parameters)
    assert params == ["ctx", "q", "k", "v", "log_fgate", "seq_start", "causal", "sm_scale", "adaptive_threshold",
                      "return_log_normalizer", "return_start_index", "record_time_key", "record_attention_time",
                      "record_find_index_time"]
    sig = inspect.signature(forgetting_attention)
    assert [p for p in sig.parameters] == ["q", "k", "v", "log_fgate", "head_first", "seq_start", "sm_scale", "adaptive_threshold"]
    assert all(sig.parameters[p].kind is inspect.Parameter.KEYWORD_ONLY for p in ("head_first", "seq_start", "sm_scale", "adaptive_threshold"))


def test_noalloc_rejects_shapes_beyond_its_array():
    """The entry point that allocates nothing holds 64 MiB for key-split partials; a shape that needs more is refused
    before anything touches the GPU."""
    lib = _lib.load()
    dims = _lib.Dims(7, 73, 128, 4096, 128, _lib.DTYPE_BF16)   # 511 query tiles x 2 splits: 68.0 MB > 64 MiB
    need = C.c_int64(0)
    _lib.check(lib.fox_attn_fwd_workspace_bytes(C.byref(dims), C.byref(need)), "fox_attn_fwd_workspace_bytes")
    assert need.value > 64 << 20
    args = _lib.FwdArgs(dims)
    rc = lib.fox_attn_fwd_noalloc(C.byref(args), None)
    assert rc == -1 and b"64" in lib.fox_last_error() and b"scratch" in lib.fox_last_error()
