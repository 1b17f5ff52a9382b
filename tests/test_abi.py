"""Host-side checks that need no GPU: the C-ABI library loads, exports every
symbol the header declares, validates arguments before touching HIP, and the
Python operator layer mirrors the reference's surface and error behaviour."""
import ctypes
import os
import re

import pytest
import torch

import proteusai_amd as pa
from proteusai_amd import _lib, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header_name):
    header = open(os.path.join(ROOT, "include", header_name)).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = sorted(set(re.findall(r"\b(proteus_[a-z0-9_]+)\s*\(", header)))
    assert declared, f"no declarations found in {header_name}"
    return declared


def test_library_exports_every_declared_symbol():
    declared = _declared("proteus_hip.h")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in proteus_hip.h but not exported"
    assert sorted(declared) == sorted(_lib.SYMBOLS)
    # the measurement probes are not part of the product library or its header
    assert not [n for n in declared if "probe" in n]
    assert not hasattr(lib, "proteus_probe_valu_rate")


def test_probe_library_exports_every_declared_symbol():
    from proteusai_amd import _probes
    declared = _declared("proteus_probes.h")
    lib = ctypes.CDLL(_probes.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in proteus_probes.h but not exported"
    assert sorted(declared) == sorted(_probes.SYMBOLS)
    # argument errors come back before any HIP call
    _probes.load()
    assert _probes.load().proteus_probe_trans_valu_mix(3, 4, 256, 10, 10, None, None, None) < 0
    assert _probes.load().proteus_probe_valu_rate(0, 1, 1, None, None) < 0


def test_version_and_strerror():
    lib = _lib.load()
    # the binding and the header agree on the version whose argument lists they describe, and the library reports it
    header = open(os.path.join(ROOT, "include", "proteus_hip.h")).read()
    assert int(re.search(r"#define\s+PROTEUS_VERSION\s+(\d+)", header).group(1)) == _lib.ABI_VERSION == lib.proteus_version()
    assert lib.proteus_strerror(0) == b"ok"
    for code in range(-9, 0):
        assert lib.proteus_strerror(code) not in (b"", b"unknown error code")
    assert lib.proteus_strerror(-99) == b"unknown error code"


def test_we_argument_validation_happens_before_any_hip_call():
    lib = _lib.load()
    p = 0x1000  # an aligned, never dereferenced address
    ok = dict(coords=p, layout=0, wn=p, mask=None, out=p, cs=p, ss=p, Z=1, N=8, K=4, tuning=0)

    def call(**kw):
        a = {**ok, **kw}
        return lib.proteus_we_fwd_check(a["coords"], a["layout"], a["wn"], a["mask"], a["out"], a["cs"], a["ss"],
                                        a["Z"], a["N"], a["K"], a["tuning"])
    assert call() == 0
    for name in ("coords", "wn", "out", "cs", "ss"):
        assert call(**{name: None}) == -1
    assert call(cs=None, ss=None) == 0                # both sums absent: the variant that does not compute them
    for name in ("Z", "N", "K"):
        assert call(**{name: 0}) == -2 and call(**{name: -3}) == -2
    assert call(N=(1 << 22) + 1) == -2 and call(K=4097) == -2
    assert call(layout=2) == -4
    assert call(out=p + 4) == -5
    assert call(tuning=999) == -6 and call(tuning=-1) == -6
    # the launching entry point runs the same checks first: a bad argument never reaches the GPU
    assert lib.proteus_we_fwd(None, 0, p, None, p, p, p, 1, 8, 4, 0, None) == -1
    assert lib.proteus_we_fwd(p, 7, p, None, p, p, p, 1, 8, 4, 0, None) == -4


def test_we_aniso_argument_validation():
    lib = _lib.load()
    p = 0x1000
    ok = dict(a=p, b=p, layout=1, cb=p, wn=p, mask=None, out=p, dcb=p, dk=p, Z=1, N=8, K=4, tuning=0)

    def call(**kw):
        a = {**ok, **kw}
        return lib.proteus_we_aniso_fwd_check(a["a"], a["b"], a["layout"], a["cb"], a["wn"], a["mask"],
                                              a["out"], a["dcb"], a["dk"], a["Z"], a["N"], a["K"], a["tuning"])
    assert call() == 0
    for name in ("a", "b", "cb", "wn", "out", "dcb", "dk"):
        assert call(**{name: None}) == -1
    assert call(dcb=None, dk=None) == 0               # only the embedding is wanted: both partials absent, not one
    for name in ("Z", "N", "K"):
        assert call(**{name: 0}) == -2
    assert call(N=(1 << 22) + 1) == -2 and call(K=4097) == -2
    assert call(layout=5) == -4
    assert call(dk=p + 8) == -5
    assert call(tuning=len(_lib.we_aniso_variants())) == -6
    assert lib.proteus_we_aniso_fwd(p, None, 1, p, p, None, p, p, p, 1, 8, 4, 0, None) == -1
    assert _lib.we_aniso_variants()[0] == "auto"


def test_attention_argument_validation():
    lib = _lib.load()
    p = 0x1000
    ok = [p, p, p, p, p, None, p, p, 1, 2, 16, 64, 0]

    def call(idx=None, val=None):
        a = list(ok)
        if idx is not None:
            a[idx] = val
        return lib.proteus_geo_attn_fwd_check(*a)
    assert call() == 0
    for idx in (0, 1, 2, 3, 4, 6):
        assert call(idx, None) == -1
    assert call(7, None) == 0                  # L is optional
    for idx in (8, 9, 10):
        assert call(idx, 0) == -2
    assert call(11, 32) == 0 and call(11, 128) == 0          # head dimensions 32, 64, 128
    assert call(11, 48) == -3 and call(11, 16) == -3 and call(11, 256) == -3
    assert call(12, 55) == -6
    assert call(0, p + 2) == -5
    assert lib.proteus_geo_attn_fwd(p, p, p, p, p, None, p, p, 1, 2, 16, 48, 0, None) == -3
    # legacy-logits entry point: same checks, plus beta and the rbf range
    assert lib.proteus_geo_attn_legacy_fwd(p, p, p, p, p, None, None, p, p, 1, 2, 16, 64, 0.0, 1.0, 0, 0, None) == -1
    assert lib.proteus_geo_attn_legacy_fwd(p, p, p, p, p, p, None, p, p, 1, 2, 16, 64, 0.5, 0.5, 0, 0, None) == -2
    assert lib.proteus_geo_attn_legacy_fwd(p, p, p, p, p, p, None, p, p, 1, 2, 16, 48, 0.0, 1.0, 0, 0, None) == -3
    # ... and the operand type: bf16 (0) or fp16 (1)
    assert lib.proteus_geo_attn_legacy_fwd(p, p, p, p, p, p, None, p, p, 1, 2, 16, 64, 0.0, 1.0, 2, 0, None) == -9
    assert lib.proteus_geo_attn_legacy_fwd(p, p, p, p, p, p, None, p, p, 1, 2, 16, 64, 0.0, 1.0, -1, 0, None) == -9


def test_attention_backward_argument_validation():
    lib = _lib.load()
    p = 0x1000
    ok = [p, p, p, p, p, p, None, None, p, p, p, p, p, p, None, 1, 2, 16, 64, 0.0, 1.0, 0]

    def call(**kw):
        a = list(ok)
        for i, v in kw.items():
            a[int(i[1:])] = v
        return lib.proteus_geo_attn_bwd_check(*a)
    assert call() == 0
    for i in (0, 1, 2, 3, 4, 5, 8, 9, 10, 11, 12):
        assert call(**{f"a{i}": None}) == -1
    assert call(a15=0) == -2 and call(a17=(1 << 20) + 1) == -2
    assert call(a18=32) == 0 and call(a18=128) == 0 and call(a18=48) == -3
    assert call(a21=1) == -9 and call(a21=2) == -9      # fp16 operands go with the legacy logits (beta) only
    assert call(a6=p, a21=1) == 0 and call(a6=p, a21=2) == -9
    assert call(a10=p + 4) == -5
    assert call(a6=p, a19=0.5, a20=0.5) == -2          # legacy logits need max_rbf > min_rbf
    assert lib.proteus_geo_attn_bwd(*(ok[:3] + [None] + ok[4:] + [None])) == -1


def test_check_raises_python_exceptions():
    with pytest.raises(ValueError):
        _lib.check(-2, "x")
    with pytest.raises(_lib.ProteusError):
        _lib.check(700, "x")
    _lib.check(0, "x")


def test_variant_tables():
    assert _lib.we_variants()[0] == "auto" and len(_lib.we_variants()) == _lib.load().proteus_we_num_variants()
    assert _lib.geo_attn_variants()[0] == "auto"
    assert _lib.load().proteus_we_variant_name(10 ** 6) is None


def test_operators_refuse_cpu_tensors_instead_of_falling_back():
    coords = torch.randn(1, 8, 3)
    with pytest.raises(_lib.ProteusError):
        pa.we_forward(coords, torch.rand(4))
    with pytest.raises(_lib.ProteusError):
        pa.wf_embedding(coords, torch.rand(4), mask=torch.zeros(1, 8, dtype=torch.bool))
    Q = torch.randn(1, 2, 8, 64)
    with pytest.raises(_lib.ProteusError):
        pa.geo_attn(Q, Q, Q, coords, torch.ones(2))


def test_operator_argument_errors_match_the_reference_surface():
    coords = torch.randn(1, 8, 3)
    with pytest.raises(ValueError):
        pa.we_forward(torch.randn(1, 8, 2), torch.rand(4))
    with pytest.raises(AssertionError):
        pa.wf_embedding(coords, torch.rand(4), magnitude_type=5)
    with pytest.raises(_lib.ProteusError):
        pa.wf_embedding(coords, torch.rand(4), magnitude_type=0)      # exists, but not on the CPU
    with pytest.raises(_lib.ProteusError):
        pa.wf_embedding(coords, torch.rand(4), dropout_p=0.1)              # exists, but not on the CPU
    with pytest.raises(ValueError):
        pa.wf_embedding(coords, torch.rand(4), dropout_p=1.0)              # the reference would divide by zero
    lib = _lib.load()
    # the dropout entry point validates before any HIP call
    assert lib.proteus_we_dropout_fwd(0x1000, 0, 0x1000, None, 0x1000, 0x1000, 0x1000, 1, 8, 4, 1, 1.5, 7, None) == -2
    assert lib.proteus_we_dropout_fwd(0x1000, 0, 0x1000, None, 0x1000, None, None, 1, 8, 4, 1, 0.5, 7, None) == -1
    assert lib.proteus_we_dropout_fwd(0x1000, 0, 0x1000, None, 0x1000, 0x1000, 0x1000, 1, 8, 4, 9, 0.5, 7, None) == -7
    assert lib.proteus_we_dropout_threshold(0.0) == 0 and lib.proteus_we_dropout_threshold(0.5) == 2 ** 31 - 64
    assert lib.proteus_we_legacy_fwd(0x1000, 0, 0x1000, None, 0x1000, 0x1000, 0x1000, 1, 8, 4, 4, None) == -7
    assert lib.proteus_we_legacy_fwd(0x1000, 0, 0x1000, None, None, 0x1000, 0x1000, 1, 8, 4, 2, None) == -1
    # the other source weights have no variant without the sums
    assert lib.proteus_we_legacy_fwd(0x1000, 0, 0x1000, None, 0x1000, None, None, 1, 8, 4, 2, None) == -1
    Q = torch.randn(1, 2, 8, 64)
    with pytest.raises(AssertionError):
        pa.geo_attn(Q, Q[:, :, :4], Q, coords, torch.ones(2))
    with pytest.raises(AssertionError):
        pa.geo_attn(Q, Q, Q, coords[:, :, :2], torch.ones(2))
    with pytest.raises(AssertionError):
        pa.geo_attn(Q, Q, Q, coords, torch.ones(3))
    with pytest.raises(NotImplementedError):
        pa.geometric_attn(Q, Q, Q, coords, torch.ones(2), None, min_rbf=0.1)     # the pair mask needs betas
    with pytest.raises(_lib.ProteusError):
        pa.geometric_attn(Q, Q, Q, coords, torch.ones(2), betas=torch.ones(2))    # legacy logits exist, but not on the CPU
    # the operator on a fused projection: qkv is [Z,N,3,H,d]
    qkv = torch.randn(1, 8, 3, 2, 64)
    with pytest.raises(AssertionError):
        pa.geometric_attn_qkv(qkv[:, :, :2], coords, torch.ones(2))
    with pytest.raises(AssertionError):
        pa.geometric_attn_qkv(qkv[0], coords, torch.ones(2))
    with pytest.raises(NotImplementedError):
        pa.geometric_attn_qkv(qkv, coords, torch.ones(2), None, max_rbf=0.9)
    with pytest.raises(_lib.ProteusError):
        pa.geometric_attn_qkv(qkv, coords, torch.ones(2))                         # not on the CPU
    # the encoder layer's add + LayerNorm is the torch expression itself for tensors the kernel does not take (CPU tensors here;
    # the two O(N^2) operators around it have no CPU path and raise)
    from proteusai_amd.encoder import add_layer_norm
    norm = torch.nn.LayerNorm(16)
    x, r = torch.randn(3, 16), torch.randn(3, 16)
    with torch.no_grad():
        assert torch.equal(add_layer_norm(x, r, norm), norm(x + r))


def test_wavefunction_embedding_module_schedule_and_parameters():
    # utils/model_utils/wf_embedding/wf_embedding.py:30-37: logspace(0,1,K,base) is endpoint inclusive
    m = pa.WaveFunctionEmbedding(d_wf=512, min_wl=3.7, max_wl=20.0, base_wl=20.0, anisotropic=False, learn_wl=True)
    wl = 2 * torch.pi / m.get_wavenumbers()
    assert wl.shape == (256,)
    assert wl[0].item() == pytest.approx(3.7, rel=1e-5) and wl[-1].item() == pytest.approx(20.0, rel=1e-5)
    assert torch.all(wl[1:] > wl[:-1])
    assert m.wavenumbers.requires_grad and not m.aa_magnitudes.requires_grad
    assert set(dict(m.named_parameters())) == {"wavenumbers", "aa_magnitudes"}
    # the default module is the anisotropic one: it needs coords_beta and, like every operator, the GPU
    with pytest.raises(ValueError):
        pa.WaveFunctionEmbedding()(torch.randn(1, 4, 3))
    with pytest.raises(_lib.ProteusError):
        pa.WaveFunctionEmbedding()(torch.randn(1, 4, 3), torch.randn(1, 4, 3))
    with pytest.raises(ValueError):
        pa.wf_embedding_learnCB(torch.randn(1, 4, 3), torch.randn(1, 5, 3), torch.ones(3), torch.ones(3))
    with pytest.raises(ValueError):
        pa.wf_embedding_learnCB(torch.randn(1, 4, 3), torch.randn(1, 4, 3), torch.ones(2), torch.ones(3))


def test_geo_attention_module_parameters():
    m = pa.GeoAttention(d_model=512, heads=8, min_spread=2.0)
    names = set(dict(m.named_parameters()))
    assert names == {"spread_weights", "beta_weights", "q_proj", "k_proj", "v_proj", "q_bias", "k_bias", "v_bias", "out_proj.weight"}
    assert tuple(m.q_proj.shape) == (8, 512, 64)
    assert torch.allclose(m.get_spreads(), torch.full((8,), 3.0))
    with pytest.raises(ValueError):
        pa.GeoAttention(d_model=100, heads=8)


def test_synthetic_inputs():
    g = torch.Generator().manual_seed(0)
    x = synth.random_walk_chain(500, g)
    bonds = (x[1:] - x[:-1]).double().norm(dim=1)
    assert torch.allclose(bonds, torch.full_like(bonds, 3.8), atol=1e-3)
    y = synth.compact_chain(x, g)
    assert synth.radius_of_gyration(y) == pytest.approx(2.2 * 500 ** 0.38, rel=1e-4)
    wl = synth.wavelength_schedule(512)
    assert wl[0].item() == pytest.approx(3.7) and wl[-1].item() < 20.0 and wl.shape == (256,)
    s = synth.log_spaced_sigma(8)
    assert s[0].item() == pytest.approx(3.0) and s[-1].item() == pytest.approx(25.0)
    c1, w1 = synth.we_inputs(64, 5)
    c2, w2 = synth.we_inputs(64, 5)
    assert torch.equal(c1, c2) and torch.equal(w1, w2)
    Q, K, V, c, sg, m = synth.attn_inputs(2, 2, 100, 64, 3, min_len=50)
    assert Q.dtype == torch.bfloat16 and m.shape == (2, 100) and (~m).sum(1).min() >= 50


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_we_backward_argument_validation_happens_before_any_hip_call():
    lib = _lib.load()
    p = 0x1000
    need = lib.proteus_we_bwd_workspace_bytes(2, 100, 16)
    assert need >= 2 * 16 * 4 and lib.proteus_we_bwd_workspace_bytes(0, 100, 16) == 0
    # the workspace grows with the rows only up to a fixed number of slabs
    assert lib.proteus_we_bwd_workspace_bytes(1, 1 << 22, 16) == lib.proteus_we_bwd_workspace_bytes(1, 1 << 20, 16)
    ok = lib.proteus_we_bwd_check(p, p, p, p, p, need, 2, 100, 16)
    assert ok == 0
    assert lib.proteus_we_bwd_check(None, p, p, p, p, need, 2, 100, 16) == -1
    assert lib.proteus_we_bwd_check(p, None, p, p, p, need, 2, 100, 16) == -1
    assert lib.proteus_we_bwd_check(p, p, p, None, p, need, 2, 100, 16) == -1
    assert lib.proteus_we_bwd_check(p, p, p, p, None, need, 2, 100, 16) == -1
    assert lib.proteus_we_bwd_check(p, p, p, p, p, need - 1, 2, 100, 16) == -2
    assert lib.proteus_we_bwd_check(p, p, p, p, p, need, 0, 100, 16) == -2
    assert lib.proteus_we_bwd_check(p, p, p, p, p, need, 2, 100, 4097) == -2
    assert lib.proteus_we_bwd_check(p + 4, p, p, p, p, need, 2, 100, 16) == -5
    assert lib.proteus_we_bwd(None, p, p, p, p, need, 2, 100, 16, None) == -1
    # anisotropic: each gradient comes with its partials or not at all; at least one is wanted
    assert lib.proteus_we_aniso_bwd_check(p, p, p, p, p, p, need, 2, 100, 16) == 0
    assert lib.proteus_we_aniso_bwd_check(p, p, None, p, None, p, need, 2, 100, 16) == 0
    assert lib.proteus_we_aniso_bwd_check(p, None, p, None, p, p, need, 2, 100, 16) == 0
    assert lib.proteus_we_aniso_bwd_check(p, p, None, p, p, p, need, 2, 100, 16) == -1
    assert lib.proteus_we_aniso_bwd_check(p, None, None, None, None, p, need, 2, 100, 16) == -1
    assert lib.proteus_we_aniso_bwd_check(p, p, p, p, p, p, need - 4, 2, 100, 16) == -2
    assert lib.proteus_we_aniso_bwd(p, p, p, p, p, None, need, 2, 100, 16, None) == -1


def test_strided_attention_argument_validation():
    import ctypes
    lib = _lib.load()
    p = 0x1000
    Z, H, N = 2, 4, 100

    def arr(*v):
        return (ctypes.c_int64 * len(v))(*v)
    plain = [H * N * 64, N * 64, 64]
    fused = [N * 3 * H * 64, 64, 3 * H * 64]                    # slices of [Z,N,3,H,d]
    tok = [N * H * 64, 64, H * 64]                             # [Z,N,H,d]

    def fwd(st):
        return lib.proteus_geo_attn_fwd_strided_check(p, p, p, st, p, p, None, p, p, Z, H, N, 64, 0)
    assert fwd(arr(*(plain * 4))) == 0
    assert fwd(arr(*(fused * 3 + tok))) == 0
    assert fwd(None) == -1
    assert fwd(arr(*(plain * 3 + [H * N * 64, N * 64, 32]))) == -4       # rows would overlap
    assert fwd(arr(*([-1, N * 64, 64] + plain * 3))) == -4
    assert fwd(arr(*([0, N * 64, 64] + plain * 3))) == -4                # batch items on top of each other
    assert fwd(arr(*([H * N * 64, N * 64, 68] + plain * 3))) == -5       # bf16 rows off 16-byte alignment
    assert fwd(arr(*(plain * 3 + [H * N * 64, N * 64, 66]))) == -5       # f32 rows off 16-byte alignment
    assert fwd(arr(*([H * N * 64, N * 64, 1 << 29] + plain * 3))) == -2  # offsets beyond 31 bits
    assert lib.proteus_geo_attn_fwd_strided(None, p, p, arr(*(plain * 4)), p, p, None, p, p, Z, H, N, 64, 0, None) == -1

    def bwd(st):
        return lib.proteus_geo_attn_bwd_strided_check(p, p, p, p, st, p, p, None, None, p, p, p, p, p, p, None,
                                                      Z, H, N, 64, 0.0, 1.0, 0)
    assert bwd(arr(*(plain * 7))) == 0
    assert bwd(arr(*(fused * 3 + tok * 4))) == 0
    assert bwd(None) == -1
    assert bwd(arr(*(plain * 6 + [H * N * 64, N * 64, 63]))) == -4
    assert bwd(arr(*(plain * 6 + [H * N * 64, N * 64, 66]))) == -5


def test_add_layernorm_argument_validation():
    lib = _lib.load()
    p = 0x1000
    f32, bf16 = _lib.DTYPE_F32, _lib.DTYPE_BF16

    def chk(x=p, res=p, gamma=p, beta=p, out=p, rows=10, D=512, eps=1e-5, dtype=bf16):
        return lib.proteus_add_layernorm_fwd_check(x, res, gamma, beta, out, rows, D, eps, dtype)
    assert chk() == 0 and chk(dtype=f32) == 0
    assert chk(res=None, gamma=None, beta=None) == 0                 # plain normalisation
    assert chk(out=p, x=p) == 0                                      # in place
    assert chk(x=None) == -1 and chk(out=None) == -1
    assert chk(dtype=2) == -9
    assert chk(rows=0) == -2 and chk(D=0) == -2
    assert chk(D=4096) == 0 and chk(D=4104) == -2                    # bf16: at most 4096
    assert chk(D=2048, dtype=f32) == 0 and chk(D=2052, dtype=f32) == -2
    assert chk(D=516) == -2 and chk(D=516, dtype=f32) == 0           # multiples of 8 (bf16), 4 (fp32)
    assert chk(eps=-1.0) == -2 and chk(eps=float("nan")) == -2
    assert chk(x=p + 8) == -5 and chk(gamma=p + 4) == -5
    assert lib.proteus_add_layernorm_fwd(None, p, p, p, p, 10, 512, 1e-5, bf16, None) == -1


def test_attention_delta_argument_validation():
    import ctypes
    lib = _lib.load()
    p = 0x1000

    def arr(*v):
        return (ctypes.c_int64 * len(v))(*v)

    def chk(O=p, dO=p, strides=None, D=p, Z=2, H=4, N=100, d=64, dtype=_lib.DTYPE_BF16):
        return lib.proteus_geo_attn_delta_check(O, dO, strides, D, Z, H, N, d, dtype)
    assert chk() == 0 and chk(dtype=_lib.DTYPE_F32) == 0 and chk(dtype=_lib.DTYPE_F16) == 0
    assert chk(O=None) == -1 and chk(dO=None) == -1 and chk(D=None) == -1
    assert chk(d=48) == -3 and chk(dtype=3) == -9
    assert chk(N=0) == -2 and chk(Z=70000, H=1) == -2
    assert chk(O=p + 8) == -5 and chk(dO=p + 4) == -5 and chk(dO=p + 8) == 0 and chk(dO=p + 8, dtype=_lib.DTYPE_F32) == -5
    plain = [4 * 100 * 64, 100 * 64, 64]
    tok = [100 * 4 * 64, 64, 4 * 64]
    assert chk(strides=arr(*(plain + tok))) == 0
    assert chk(strides=arr(*(plain + [4 * 100 * 64, 100 * 64, 32]))) == -4          # rows would overlap
    assert chk(strides=arr(*([-4, 100 * 64, 64] + plain))) == -4
    assert chk(strides=arr(*(plain + [4 * 100 * 64, 100 * 64, 66]))) == -5          # rows off the 4-element grid
    assert lib.proteus_geo_attn_delta(None, p, None, p, 2, 4, 100, 64, _lib.DTYPE_BF16, None) == -1
