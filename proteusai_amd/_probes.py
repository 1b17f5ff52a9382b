"""ctypes binding of libproteus_probes.so (declarations in include/proteus_probes.h): instruction-rate, accuracy and
co-issue micro-benchmarks.  Measurement only: the operators never load it; bench.py and the test of the hardware
sin/cos error do."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libproteus_probes.so")

# every symbol include/proteus_probes.h declares
SYMBOLS = ["proteus_probe_valu_rate", "proteus_probe_sincos", "proteus_probe_mfma_softmax_slot", "proteus_probe_trans_valu_mix"]

_lib = None


def load():
    """Load the probe library; raise if it has not been built (`python -m proteusai_amd.build` builds it)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m proteusai_amd.build`")
    lib = ctypes.CDLL(LIB_PATH)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.proteus_probe_valu_rate.restype = ci
    lib.proteus_probe_valu_rate.argtypes = [ci, ci, ci, vp, vp]
    lib.proteus_probe_sincos.restype = ci
    lib.proteus_probe_sincos.argtypes = [vp, vp, vp, vp, ci, ci, vp]
    lib.proteus_probe_mfma_softmax_slot.restype = ci
    lib.proteus_probe_mfma_softmax_slot.argtypes = [ci, ci, ci, vp, vp]
    lib.proteus_probe_trans_valu_mix.restype = ci
    lib.proteus_probe_trans_valu_mix.argtypes = [ci, ci, ci, ci, ci, vp, vp, vp]
    _lib = lib
    return lib
