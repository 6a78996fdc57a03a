"""ctypes binding of librexsc.so (the C ABI declared in include/rexsc.h).

The library is the only compute path: if it is missing, or an entry point fails, the caller
gets a RuntimeError -- there is no Python/CPU fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librexsc.so")
NOALLOC_SCRATCH_BYTES = 32 << 20  # REXSC_NOALLOC_SCRATCH_BYTES of include/rexsc.h
ABI_VERSION = 200                 # REXSC_ABI_VERSION of include/rexsc.h: the layout the structures below mirror
WSTREAMS_FILL, WSTREAMS_TRUST, WSTREAMS_VERIFY = 0, 1, 2  # REXSC_WSTREAMS_*
_lib = None


class _Desc(ctypes.Structure):
    """A descriptor of include/rexsc.h.  Its first field is its own size, filled here: positional arguments start
    at the field after it.  The library refuses a descriptor of any other size."""

    def __init__(self, *args, **kwargs):
        super().__init__(ctypes.sizeof(type(self)), *args, **kwargs)

    def key(self):
        return tuple(getattr(self, f[0]) for f in self._fields_)


class ConvDesc(_Desc):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "struct_size", "N", "C", "H", "W", "O", "KH", "KW", "pad_h", "pad_w", "stride_h", "stride_w",
        "bit_length", "lfsr_length", "gen_config", "bin_config",
        "total_width", "load_width", "load_wait", "act_channels_last", "weight_channels_last", "xnor",
        "act_fake_quant", "weight_fake_quant")]


class LinearDesc(_Desc):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "struct_size", "B", "C", "O", "bit_length", "lfsr_length", "gen_config", "bin_config",
        "total_width", "load_width", "load_wait", "act_fake_quant", "weight_fake_quant")]


class FixedDesc(_Desc):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "struct_size", "N", "C", "H", "W", "O", "KH", "KW", "pad_h", "pad_w", "stride_h", "stride_w",
        "add_config", "precision_in", "precision_out")]


class ProfileRecord(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("calls", ctypes.c_int32), ("total_ms", ctypes.c_double),
                ("total_work", ctypes.c_double)]


_vp = ctypes.c_void_p
_sz = ctypes.c_size_t
_int = ctypes.c_int
_u64 = ctypes.c_uint64

# name -> (restype, argtypes); every symbol include/rexsc.h declares
SIGNATURES = {
    "rexsc_last_error": (ctypes.c_char_p, []),
    "rexsc_version": (_int, []),
    "rexsc_init": (_int, [_vp]),
    "rexsc_conv2d_workspace_bytes": (_sz, [ctypes.POINTER(ConvDesc)]),
    "rexsc_conv2d_plan_info": (_int, [ctypes.POINTER(ConvDesc), ctypes.POINTER(ctypes.c_int64)]),
    "rexsc_conv2d_orn": (_int, [ctypes.POINTER(ConvDesc), _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "rexsc_conv2d_weight_streams_bytes": (_sz, [ctypes.POINTER(ConvDesc)]),
    "rexsc_conv2d_orn_ex": (_int, [ctypes.POINTER(ConvDesc), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _int, _vp, _sz, _vp]),
    "rexsc_conv2d_prepare_weights": (_int, [ctypes.POINTER(ConvDesc), _vp, _vp, _sz, _int, _vp]),
    "rexsc_conv2d_orn_noalloc": (_int, [ctypes.POINTER(ConvDesc), _vp, _vp, _vp, _vp, _vp, _vp]),
    "rexsc_linear_workspace_bytes": (_sz, [ctypes.POINTER(LinearDesc)]),
    "rexsc_linear_orn": (_int, [ctypes.POINTER(LinearDesc), _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "rexsc_linear_weight_streams_bytes": (_sz, [ctypes.POINTER(LinearDesc)]),
    "rexsc_linear_orn_ex": (_int, [ctypes.POINTER(LinearDesc), _vp, _vp, _vp, _vp, _vp, _sz, _int, _vp, _sz, _vp]),
    "rexsc_linear_legacy": (_int, [ctypes.POINTER(LinearDesc), _int, _int, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "rexsc_orn_forward": (_int, [_vp, _vp, _sz, _int, _vp]),
    "rexsc_orn_backward": (_int, [_vp, _vp, _vp, _sz, _int, _int, _vp]),
    "rexsc_orn_bias_std_both_forward": (_int, [_vp, _vp, _vp, _vp, _vp, _sz, _int, _u64, _u64, _vp, _vp, _vp, _vp]),
    "rexsc_orn_bias_std_both_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _int, _int, _vp]),
    "rexsc_orn_bias_std_forward_f16": (_int, [_vp, _vp, _vp, _vp, _sz, _int, _u64, _u64, _vp, _vp]),
    "rexsc_orn_bias_std_backward": (_int, [_vp, _vp, _vp, _vp, _sz, _int, _int, _vp]),
    "rexsc_orn_pair_backward": (_int, [_vp, _vp, _vp, _sz, _sz, _int, _int, _vp]),
    "rexsc_orn_pair_backward_f16": (_int, [_vp, _vp, _vp, _sz, _sz, _int, _vp]),
    "rexsc_orn_bias_std_pair_forward": (_int, [_vp, _vp, _vp, _vp, _sz, _sz, _int, _u64, _u64, _vp, _vp]),
    "rexsc_orn_bias_std_pair_backward": (_int, [_vp, _vp, _vp, _vp, _sz, _sz, _int, _int, _vp]),
    "rexsc_sc_counts_to_float": (_int, [_vp, _vp, _vp, _sz, _int, _vp]),
    "rexsc_split_weight": (_int, [_vp, _vp, _sz, _sz, _sz, _int, _int, _vp]),
    "rexsc_merge_weight_grad": (_int, [_vp, _vp, _vp, _sz, _sz, _sz, _int, _int, _vp]),
    "rexsc_quantize": (_int, [_vp, _vp, _sz, _int, _vp]),
    "rexsc_quantize_f16": (_int, [_vp, _vp, _sz, _int, _vp]),
    "rexsc_philox4x32_10": (None, [ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32),
                                   ctypes.POINTER(ctypes.c_uint32)]),
    "rexsc_fixed_conv2d_workspace_bytes": (_sz, [ctypes.POINTER(FixedDesc)]),
    "rexsc_fixed_conv2d": (_int, [ctypes.POINTER(FixedDesc), _vp, _vp, _vp, _vp, _sz, _vp]),
    "rexsc_profile_begin": (_int, []),
    "rexsc_profile_end": (_int, [ctypes.POINTER(ProfileRecord), _int]),
    "rexsc_valu_probe": (_int, [_int, _int, _vp, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
    "rexsc_calib_stats": (_int, [_vp, _vp, _sz, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float),
                                 _int, _vp, _vp]),
}


def lib():
    """Load librexsc.so once.  Raises RuntimeError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "librexsc.so is missing (%s): build it with `python rex-sc_amd/build.py`; "
                "there is no fallback path" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        handle.rexsc_version.restype = ctypes.c_int
        if handle.rexsc_version() != ABI_VERSION:
            raise RuntimeError("librexsc.so reports ABI version %d, this binding mirrors version %d: rebuild it with "
                               "`python rex-sc_amd/build.py --force`" % (handle.rexsc_version(), ABI_VERSION))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc, what):
    if rc != 0:
        msg = lib().rexsc_last_error()
        raise RuntimeError("%s failed (code %d): %s" % (what, rc, msg.decode() if msg else "?"))


def profile_begin():
    check(lib().rexsc_profile_begin(), "rexsc_profile_begin")


def profile_end(max_records=64):
    """-> {kernel name: dict(calls, total_ms, total_work)}"""
    buf = (ProfileRecord * max_records)()
    n = lib().rexsc_profile_end(buf, max_records)
    return {buf[i].name.decode(): dict(calls=buf[i].calls, total_ms=buf[i].total_ms, total_work=buf[i].total_work)
            for i in range(n)}


def valu_probe(mode=0, iters=2000, stream=None):
    """-> lane-ops/s sustained by the register-only AND/popcount (mode 0) or AND-OR (mode 1) probe kernel."""
    ms, ops = ctypes.c_double(), ctypes.c_double()
    check(lib().rexsc_valu_probe(int(mode), int(iters), stream, ctypes.byref(ms), ctypes.byref(ops)), "rexsc_valu_probe")
    return ops.value / (ms.value * 1e-3)
