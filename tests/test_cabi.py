"""The C-ABI library loads and exports every symbol include/rexsc.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "rexsc.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rexsc_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_entry_points():
    names = _declared()
    for must in ("rexsc_conv2d_orn", "rexsc_linear_orn", "rexsc_orn_forward", "rexsc_orn_backward",
                 "rexsc_orn_bias_std_both_forward", "rexsc_orn_bias_std_both_backward", "rexsc_fixed_conv2d",
                 "rexsc_calib_stats", "rexsc_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    import _lib
    handle = _lib.lib()
    for name in _declared():
        assert hasattr(handle, name), "librexsc.so lacks " + name
    # and the ctypes table binds exactly the declared set
    assert sorted(_lib.SIGNATURES) == _declared()


def test_planning_and_errors_need_no_gpu():
    import _lib
    L = _lib.lib()
    header = open(os.path.join(ROOT, "include", "rexsc.h")).read()
    assert L.rexsc_version() == _lib.ABI_VERSION == int(re.search(r"#define REXSC_ABI_VERSION (\d+)", header).group(1))
    d = _lib.ConvDesc(64, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 32, -1, 1, 1, 7, 8, 1, 1, 0)
    assert L.rexsc_conv2d_workspace_bytes(ctypes.byref(d)) > 32 * 64 * 58 * 58 * 2 * 4
    bad = _lib.ConvDesc(64, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 48, -1, 1, 1, 7, 8, 1, 1, 0)  # L=48 unsupported
    assert L.rexsc_conv2d_workspace_bytes(ctypes.byref(bad)) == 0
    assert b"stream length" in L.rexsc_last_error()
    big = _lib.ConvDesc(1, 8192, 12, 12, 4, 9, 9, 0, 0, 1, 1, 32, -1, 1, 1, 7, 8, 1, 0, 0)  # 32*81*256 >= 65536
    assert L.rexsc_conv2d_workspace_bytes(ctypes.byref(big)) == 0
    assert b"reduction too large" in L.rexsc_last_error()
    ld = _lib.LinearDesc(256, 4096, 1024, 64, -1, 1, 1, 7, 8, 1)
    assert L.rexsc_linear_workspace_bytes(ctypes.byref(ld)) > 0
    fd = _lib.FixedDesc(2, 8, 6, 6, 4, 3, 3, 1, 1, 1, 1, 0, 5, 24)
    assert L.rexsc_fixed_conv2d_workspace_bytes(ctypes.byref(fd)) > 0


def test_descriptor_of_another_abi_is_rejected():
    """Every descriptor starts with its own size; one built against another header (here: three int32 fields short,
    the conv descriptor of ABI 100) is refused instead of being read past its end."""
    import _lib
    L = _lib.lib()
    d = _lib.ConvDesc(64, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 32, -1, 1, 1, 7, 8, 1, 1, 0)
    assert d.struct_size == ctypes.sizeof(_lib.ConvDesc) == 24 * 4
    d.struct_size -= 12
    assert L.rexsc_conv2d_workspace_bytes(ctypes.byref(d)) == 0
    assert b"struct_size" in L.rexsc_last_error()
    out = (ctypes.c_int64 * 16)()
    assert L.rexsc_conv2d_plan_info(ctypes.byref(d), out) == -1
    ld = _lib.LinearDesc(256, 4096, 1024, 64, -1, 1, 1, 7, 8, 1)
    assert ld.struct_size == 13 * 4 and ld.weight_fake_quant == 0
    ld.struct_size = 0
    assert L.rexsc_linear_workspace_bytes(ctypes.byref(ld)) == 0 and b"struct_size" in L.rexsc_last_error()
    fd = _lib.FixedDesc(2, 8, 6, 6, 4, 3, 3, 1, 1, 1, 1, 0, 5, 24)
    fd.struct_size += 4
    assert L.rexsc_fixed_conv2d_workspace_bytes(ctypes.byref(fd)) == 0 and b"struct_size" in L.rexsc_last_error()
    # the ctypes mirrors have as many int32 fields as the header's structures
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "rexsc.h")).read(), flags=re.S)
    for name, cls in (("rexsc_conv_desc", _lib.ConvDesc), ("rexsc_linear_desc", _lib.LinearDesc),
                      ("rexsc_fixed_desc", _lib.FixedDesc)):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), text, flags=re.S).group(1)
        fields = [f.strip() for decl in re.findall(r"int32_t([^;]*);", body) for f in decl.split(",")]
        assert fields == [f[0] for f in cls._fields_], name


def test_philox_known_answers():
    """Philox4x32-10 vectors published with Random123 (kat_vectors)."""
    import _lib
    L = _lib.lib()
    U4 = ctypes.c_uint32 * 4
    U2 = ctypes.c_uint32 * 2
    kats = [
        ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
        ((0xffffffff,) * 4, (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
        ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
         (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
    ]
    for ctr, key, want in kats:
        out = U4()
        L.rexsc_philox4x32_10(U4(*ctr), U2(*key), out)
        assert tuple(out) == want


def test_ops_fail_loudly_without_the_library(monkeypatch, tmp_path):
    import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_product_never_touches_the_oracle():
    """The oracle is test infrastructure: nothing under the package, and none of the product's entry
    modules, may import, load or run anything under oracle/ (bench.py may, for its CPU baseline only;
    __graft_entry__ may, to build it and inside smoke())."""
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pkg = os.path.join(root, "rex-sc_amd")
    pat = re.compile(r"oracle|rexsc_oracle|_ref\b")
    offenders = []
    for dirpath, _, files in os.walk(pkg):
        if os.path.basename(dirpath) in ("build", "__pycache__"):
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f), encoding="utf-8", errors="replace").read()
                for n, line in enumerate(text.splitlines(), 1):
                    # the two names of the xnor modes are not references to the oracle directory
                    if pat.search(line.replace("cpu_oracle", "").replace("cuda_ref", "")):
                        offenders.append("%s:%d: %s" % (os.path.relpath(os.path.join(dirpath, f), root), n, line.strip()))
    assert not offenders, "\n".join(offenders)
    extra = open(os.path.join(root, "bench_extra.py")).read()
    assert "oracle" not in extra
