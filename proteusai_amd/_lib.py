"""ctypes binding of libproteus_hip.so (declarations in include/proteus_hip.h).

There is no CPU fallback: if the library is missing or a call fails, an
exception is raised.
"""
import ctypes
import functools
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libproteus_hip.so")

COORDS_SOA = 0
COORDS_AOS = 1
ABI_VERSION = 301                    # PROTEUS_VERSION of the include/proteus_hip.h these argument lists were written from
OPERAND_BF16, OPERAND_F16 = 0, 1     # PROTEUS_OPERAND_* of include/proteus_hip.h
DTYPE_F32, DTYPE_BF16, DTYPE_F16 = 0, 1, 2   # PROTEUS_DTYPE_*

# every symbol include/proteus_hip.h declares
SYMBOLS = [
    "proteus_version", "proteus_strerror",
    "proteus_we_fwd", "proteus_we_fwd_check", "proteus_we_legacy_fwd", "proteus_we_dropout_fwd", "proteus_we_dropout_fwd_check",
    "proteus_we_dropout_threshold", "proteus_we_num_variants", "proteus_we_variant_name",
    "proteus_we_aniso_fwd", "proteus_we_aniso_fwd_check", "proteus_we_aniso_num_variants", "proteus_we_aniso_variant_name",
    "proteus_we_bwd_workspace_bytes", "proteus_we_bwd", "proteus_we_bwd_check", "proteus_we_bwd_static", "proteus_we_aniso_bwd", "proteus_we_aniso_bwd_check",
    "proteus_geo_attn_fwd", "proteus_geo_attn_fwd_check", "proteus_geo_attn_legacy_fwd", "proteus_geo_attn_bwd",
    "proteus_geo_attn_fwd_workspace_bytes", "proteus_geo_attn_fwd_ws", "proteus_geo_attn_fwd_ws_check",
    "proteus_geo_attn_bwd_check", "proteus_geo_attn_fwd_strided", "proteus_geo_attn_fwd_strided_check",
    "proteus_geo_attn_legacy_fwd_strided",
    "proteus_geo_attn_bwd_strided", "proteus_geo_attn_bwd_strided_check", "proteus_geo_attn_num_variants",
    "proteus_geo_attn_variant_name",
    "proteus_add_layernorm_fwd", "proteus_add_layernorm_fwd_check", "proteus_geo_attn_delta", "proteus_geo_attn_delta_check",
]

_lib = None


class ProteusError(RuntimeError):
    pass


def load():
    """Load the HIP library; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ProteusError(
            f"{LIB_PATH} is missing: build it with `python -m proteusai_amd.build` "
            "(there is no CPU fallback)")
    lib = ctypes.CDLL(LIB_PATH)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.proteus_version.restype = ci
    if lib.proteus_version() != ABI_VERSION:
        raise ProteusError(f"{LIB_PATH} reports version {lib.proteus_version()}, this binding was written for {ABI_VERSION}: "
                           "argument lists differ between versions; rebuild with `python -m proteusai_amd.build`")
    lib.proteus_strerror.restype = ctypes.c_char_p
    lib.proteus_strerror.argtypes = [ci]
    lib.proteus_we_fwd.restype = ci
    lib.proteus_we_fwd.argtypes = [vp, ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, vp]
    lib.proteus_we_legacy_fwd.restype = ci
    lib.proteus_we_legacy_fwd.argtypes = [vp, ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, vp]
    lib.proteus_we_dropout_fwd.restype = ci
    lib.proteus_we_dropout_fwd.argtypes = [vp, ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ctypes.c_float, ctypes.c_uint32, vp]
    lib.proteus_we_dropout_fwd_check.restype = ci
    lib.proteus_we_dropout_fwd_check.argtypes = [vp, ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ctypes.c_float]
    lib.proteus_we_dropout_threshold.restype = ctypes.c_uint32
    lib.proteus_we_dropout_threshold.argtypes = [ctypes.c_float]
    lib.proteus_we_fwd_check.restype = ci
    lib.proteus_we_fwd_check.argtypes = [vp, ci, vp, vp, vp, vp, vp, ci, ci, ci, ci]
    lib.proteus_we_num_variants.restype = ci
    lib.proteus_we_variant_name.restype = ctypes.c_char_p
    lib.proteus_we_variant_name.argtypes = [ci]
    lib.proteus_we_aniso_fwd.restype = ci
    lib.proteus_we_aniso_fwd.argtypes = [vp, vp, ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, vp]
    lib.proteus_we_aniso_fwd_check.restype = ci
    lib.proteus_we_aniso_fwd_check.argtypes = [vp, vp, ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci]
    lib.proteus_we_aniso_num_variants.restype = ci
    lib.proteus_we_aniso_variant_name.restype = ctypes.c_char_p
    lib.proteus_we_aniso_variant_name.argtypes = [ci]
    sz = ctypes.c_size_t
    lib.proteus_we_bwd_workspace_bytes.restype = sz
    lib.proteus_we_bwd_workspace_bytes.argtypes = [ci, ci, ci]
    lib.proteus_we_bwd.restype = ci
    lib.proteus_we_bwd.argtypes = [vp, vp, vp, vp, vp, sz, ci, ci, ci, vp]
    lib.proteus_we_bwd_static.restype = ci
    lib.proteus_we_bwd_static.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp]
    lib.proteus_we_bwd_check.restype = ci
    lib.proteus_we_bwd_check.argtypes = [vp, vp, vp, vp, vp, sz, ci, ci, ci]
    lib.proteus_we_aniso_bwd.restype = ci
    lib.proteus_we_aniso_bwd.argtypes = [vp, vp, vp, vp, vp, vp, sz, ci, ci, ci, vp]
    lib.proteus_we_aniso_bwd_check.restype = ci
    lib.proteus_we_aniso_bwd_check.argtypes = [vp, vp, vp, vp, vp, vp, sz, ci, ci, ci]
    lib.proteus_geo_attn_fwd.restype = ci
    lib.proteus_geo_attn_fwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    lib.proteus_geo_attn_legacy_fwd.restype = ci
    lib.proteus_geo_attn_legacy_fwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci,
                                                ctypes.c_float, ctypes.c_float, ci, ci, vp]
    cf = ctypes.c_float
    lib.proteus_geo_attn_bwd.restype = ci
    lib.proteus_geo_attn_bwd.argtypes = [vp] * 15 + [ci, ci, ci, ci, cf, cf, ci, vp]
    lib.proteus_geo_attn_bwd_check.restype = ci
    lib.proteus_geo_attn_bwd_check.argtypes = [vp] * 15 + [ci, ci, ci, ci, cf, cf, ci]
    i64p = ctypes.POINTER(ctypes.c_int64)
    lib.proteus_geo_attn_fwd_strided.restype = ci
    lib.proteus_geo_attn_fwd_strided.argtypes = [vp, vp, vp, i64p, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    lib.proteus_geo_attn_fwd_strided_check.restype = ci
    lib.proteus_geo_attn_fwd_strided_check.argtypes = [vp, vp, vp, i64p, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
    lib.proteus_geo_attn_legacy_fwd_strided.restype = ci
    lib.proteus_geo_attn_legacy_fwd_strided.argtypes = [vp, vp, vp, i64p, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci,
                                                        ctypes.c_float, ctypes.c_float, ci, ci, vp]
    lib.proteus_geo_attn_bwd_strided.restype = ci
    lib.proteus_geo_attn_bwd_strided.argtypes = [vp] * 4 + [i64p] + [vp] * 11 + [ci, ci, ci, ci, cf, cf, ci, vp]
    lib.proteus_geo_attn_bwd_strided_check.restype = ci
    lib.proteus_geo_attn_bwd_strided_check.argtypes = [vp] * 4 + [i64p] + [vp] * 11 + [ci, ci, ci, ci, cf, cf, ci]
    lib.proteus_geo_attn_fwd_workspace_bytes.restype = sz
    lib.proteus_geo_attn_fwd_workspace_bytes.argtypes = [ci, ci, ci, ci, ci]
    lib.proteus_geo_attn_fwd_ws.restype = ci
    lib.proteus_geo_attn_fwd_ws.argtypes = [vp, vp, vp, i64p, vp, vp, vp, vp, vp, vp, sz, ci, ci, ci, ci, ci, vp]
    lib.proteus_geo_attn_fwd_ws_check.restype = ci
    lib.proteus_geo_attn_fwd_ws_check.argtypes = [vp, vp, vp, i64p, vp, vp, vp, vp, vp, vp, sz, ci, ci, ci, ci, ci]
    lib.proteus_geo_attn_fwd_check.restype = ci
    lib.proteus_geo_attn_fwd_check.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
    lib.proteus_geo_attn_num_variants.restype = ci
    lib.proteus_geo_attn_variant_name.restype = ctypes.c_char_p
    lib.proteus_geo_attn_variant_name.argtypes = [ci]
    lib.proteus_add_layernorm_fwd.restype = ci
    lib.proteus_add_layernorm_fwd.argtypes = [vp, vp, vp, vp, vp, ctypes.c_long, ci, cf, ci, vp]
    lib.proteus_add_layernorm_fwd_check.restype = ci
    lib.proteus_add_layernorm_fwd_check.argtypes = [vp, vp, vp, vp, vp, ctypes.c_long, ci, cf, ci]
    lib.proteus_geo_attn_delta.restype = ci
    lib.proteus_geo_attn_delta.argtypes = [vp, vp, i64p, vp, ci, ci, ci, ci, ci, vp]
    lib.proteus_geo_attn_delta_check.restype = ci
    lib.proteus_geo_attn_delta_check.argtypes = [vp, vp, i64p, vp, ci, ci, ci, ci, ci]
    _lib = lib
    return lib


def check(rc: int, what: str):
    """Turn a return code into an exception: argument errors -> ValueError,
    HIP errors -> ProteusError."""
    if rc == 0:
        return
    msg = load().proteus_strerror(rc).decode()
    if rc < 0:
        raise ValueError(f"{what}: {msg} (code {rc})")
    raise ProteusError(f"{what}: HIP error {rc}: {msg}")


def we_variants():
    lib = load()
    return [lib.proteus_we_variant_name(i).decode() for i in range(lib.proteus_we_num_variants())]


def we_aniso_variants():
    lib = load()
    return [lib.proteus_we_aniso_variant_name(i).decode() for i in range(lib.proteus_we_aniso_num_variants())]


def geo_attn_variants():
    lib = load()
    return [lib.proteus_geo_attn_variant_name(i).decode() for i in range(lib.proteus_geo_attn_num_variants())]


@functools.lru_cache(maxsize=256)
def _stride_array_of(vals):
    return (ctypes.c_int64 * len(vals))(*vals)


def stride_array(*tensors):
    """(batch, head, token) element strides of [Z,H,N,d] tensors, flattened, as the strided entry points take them
    (the arrays are read-only for the library and kept per combination of strides)."""
    vals = ()
    for t in tensors:
        vals += t.stride()[:3]
    return _stride_array_of(vals)


def raw_stream(dev):
    """Handle of torch's current stream on `dev` for the `stream` argument of the entry points."""
    import torch
    try:
        return torch._C._cuda_getCurrentRawStream(dev.index if dev.index is not None else torch.cuda.current_device())
    except AttributeError:       # (a torch without the short cut)
        return torch.cuda.current_stream(dev).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def on_device(dev):
    """Context that makes `dev` the current device for the launch; free when it already is."""
    import torch
    if dev.index is None or torch.cuda.current_device() == dev.index:
        return _NO_SWITCH
    return torch.cuda.device(dev)
