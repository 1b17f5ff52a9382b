"""GPU tests of the fused residual add + LayerNorm (proteus_add_layernorm_fwd) against the torch expression it
replaces in the encoder layer, norm(x + res) (old/old_scripts/encoder.py:36-39), evaluated on the CPU in fp64 from
the same inputs.  Bars: fp32 tensors rel-L2 <= 1e-6 and max |err| <= 1e-5; bf16 tensors within one rounding of the
result to bf16 (|err| <= 2^-8 |ref| + 2^-8 * 1e-2) of the fp64 LayerNorm of the bf16-rounded sum."""
import ctypes

import numpy as np
import pytest
import torch
import torch.nn as nn

from proteusai_amd import _lib
from proteusai_amd.encoder import add_layer_norm

pytestmark = pytest.mark.gpu


def reference(x, res, w, b, eps):
    s = x.double() if res is None else (x + res).double()          # the sum in the tensors' own type, as torch takes it
    mean = s.mean(-1, keepdim=True)
    var = ((s - mean) ** 2).mean(-1, keepdim=True)
    y = (s - mean) / torch.sqrt(var + eps)
    if w is not None:
        y = y * w.double()
    if b is not None:
        y = y + b.double()
    return y


def check(out, ref, dtype, what):
    out = out.double().cpu()
    assert torch.isfinite(out).all(), what
    err = (out - ref).abs()
    if dtype == torch.float32:
        assert float(err.max()) <= 1e-5 and float((out - ref).norm() / ref.norm()) <= 1e-6, f"{what}: {float(err.max()):.3e}"
    else:
        assert bool((err <= 2.0 ** -8 * ref.abs() + 2.0 ** -8 * 1e-2).all()), f"{what}: {float((err / (ref.abs() + 1e-2)).max()):.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,D", [(1, 512), (1001, 512), (8192, 512), (37, 128), (5, 520), (64, 2048), (3, 8), (129, 1536)])
def test_module_path_equals_the_torch_expression(gpu, dtype, rows, D):
    if dtype == torch.float32 and D % 4:
        pytest.skip("fp32 rows are multiples of 4")
    g = torch.Generator().manual_seed(rows * 7919 + D)
    x = (torch.randn(rows, D, generator=g) * 3 + 0.5).to(dtype)
    res = torch.randn(rows, D, generator=g).to(dtype)
    norm = nn.LayerNorm(D)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(D, generator=g))
        norm.bias.copy_(torch.randn(D, generator=g))
    norm = norm.to(dtype)
    ref = reference(x, res, norm.weight.detach(), norm.bias.detach(), norm.eps)
    norm_g = norm.to(gpu)
    with torch.no_grad():
        out = add_layer_norm(x.to(gpu), res.to(gpu), norm_g)
        torch_out = norm_g(x.to(gpu) + res.to(gpu))
    check(out, ref, dtype, f"rows={rows} D={D} {dtype}")
    # and against what torch itself returns on the GPU (its fp32 statistics carry their own rounding; bf16: at most
    # one rounding apart)
    tol = 1e-4 if dtype == torch.float32 else 2.0 ** -7
    worst = float(((out.double() - torch_out.double()).abs() / (torch_out.double().abs() + 1e-2)).max())
    assert worst <= tol, f"rows={rows} D={D} {dtype}: {worst:.3e} from torch's result"


def test_with_gradients_the_torch_expression_runs(gpu):
    # training: autograd differentiates the torch expression; the fused kernel is the inference path only
    x = torch.randn(4, 64, device=gpu, requires_grad=True)
    res = torch.randn(4, 64, device=gpu)
    norm = nn.LayerNorm(64).to(gpu)
    out = add_layer_norm(x, res, norm)
    out.sum().backward()
    assert x.grad is not None and torch.equal(out, norm(x + res))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_raw_c_abi_optional_pointers_and_in_place(gpu, dtype):
    lib = _lib.load()
    code = _lib.DTYPE_F32 if dtype == torch.float32 else _lib.DTYPE_BF16
    rows, D = 300, 4096 if dtype == torch.bfloat16 else 2048
    g = torch.Generator().manual_seed(5)
    x = torch.randn(rows, D, generator=g).to(dtype)
    res = torch.randn(rows, D, generator=g).to(dtype)
    w = torch.randn(D, generator=g).to(dtype)
    b = torch.randn(D, generator=g).to(dtype)
    xg, rg, wg, bg = x.to(gpu), res.to(gpu), w.to(gpu), b.to(gpu)
    st = torch.cuda.current_stream().cuda_stream
    for use_res, use_w, use_b in [(True, True, True), (False, True, True), (True, False, False), (True, True, False), (False, False, True)]:
        out = torch.full_like(xg, float("nan"))
        rc = lib.proteus_add_layernorm_fwd(xg.data_ptr(), rg.data_ptr() if use_res else None, wg.data_ptr() if use_w else None,
                                           bg.data_ptr() if use_b else None, out.data_ptr(), rows, D, 1e-5, code, st)
        assert rc == 0
        ref = reference(x, res if use_res else None, w if use_w else None, b if use_b else None, 1e-5)
        check(out, ref, dtype, f"res={use_res} gamma={use_w} beta={use_b} {dtype}")
    # in place over x
    xin = xg.clone()
    assert lib.proteus_add_layernorm_fwd(xin.data_ptr(), rg.data_ptr(), wg.data_ptr(), bg.data_ptr(), xin.data_ptr(), rows, D, 1e-5, code, st) == 0
    check(xin, reference(x, res, w, b, 1e-5), dtype, f"in place {dtype}")


def test_constant_rows_and_large_offsets(gpu):
    # a constant row has variance 0: the result is beta; a large common offset must not leak into the variance
    D = 512
    x = torch.full((2, D), 3.0)
    x[1] = torch.randn(D, generator=torch.Generator().manual_seed(1)) * 1e-2 + 1000.0
    res = torch.zeros(2, D)
    norm = nn.LayerNorm(D)
    with torch.no_grad():
        norm.bias.fill_(0.25)
    ref = reference(x, res, norm.weight.detach(), norm.bias.detach(), norm.eps)
    with torch.no_grad():
        out = add_layer_norm(x.to(gpu), res.to(gpu), norm.to(gpu))
    assert torch.equal(out[0].cpu(), torch.full((D,), 0.25))
    # (the fp32 sum of 512 values near 1000 is good to about 0.03, the mean to 6e-5: 6e-3 of the row's 1e-2 spread)
    assert float((out[1].double().cpu() - ref[1]).abs().max()) <= 2e-2
