"""Host-side checks of the C ABI that need no GPU: the library loads, exports
every symbol include/ixhip.h declares, and refuses malformed requests before
any kernel launch."""
import ctypes as C
import os
import re

import pytest
import torch

from ixrun_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header="ixhip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ixh_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    lib = _lib.lib()
    names = declared_symbols()
    assert "ixh_gemv" in names and "ixh_decode" in names and "ixh_prefix_build" in names
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/ixhip.h but not exported"
    assert set(_lib.EXPORTS) == set(names)
    assert lib.ixh_version() >= 100


def test_option_setter_is_not_in_the_product_header():
    """The process-wide kernel-selection switches are a testing hook: the product header declares no setter (nor
    mentions one), the test header declares exactly that one symbol, and the binding reads nothing from the
    environment but the library's path."""
    public = open(os.path.join(ROOT, "include", "ixhip.h")).read()
    assert "set_option" not in public and "option" not in " ".join(declared_symbols())
    assert declared_symbols("ixhip_test.h") == ["ixh_set_option"] == list(_lib.TEST_EXPORTS)
    assert hasattr(_lib.lib(), "ixh_set_option")
    pkg = os.path.join(ROOT, "ixrun_amd")
    reads = []
    for name in sorted(os.listdir(pkg)):
        if name.endswith(".py"):
            text = open(os.path.join(pkg, name)).read()
            reads += [(name, var) for var in re.findall(r"environ(?:\.get)?[\[(]\s*\"([A-Z_0-9]+)\"", text)]
    assert reads == [("_lib.py", "IXH_LIB")], reads


def _packed(level_bits=(3, 5, 8), out_f=4, in_f=8, bm0_words=1):
    s = _lib.IxhPacked()
    s.n_levels = len(level_bits)
    for i, b in enumerate(level_bits):
        s.level_bits[i] = b
    s.out_f, s.in_f = out_f, in_f
    s.bitmaps[0] = 0x1000
    s.bitmap_words[0] = bm0_words
    s.scale = 0x1000
    return s


def test_entries_and_workspace_sizes():
    lib = _lib.lib()
    assert lib.ixh_prefix_entries(10, 5) == 3 and lib.ixh_prefix_entries(11, 5) == 4
    assert lib.ixh_prefix_entries(0, 512) == 1 and lib.ixh_prefix_entries(10, 0) == -1
    s = _packed(out_f=8, in_f=2048, bm0_words=512)
    assert lib.ixh_gemv_workspace_bytes(C.byref(s), 512, 3, 0) == 4 * 3 * 8 * 4
    assert lib.ixh_gemv_workspace_bytes(C.byref(s), 2048, 3, 0) == 0
    assert lib.ixh_gemv_workspace_bytes(C.byref(s), 512, 3, _lib.IXH_GEMV_ATOMIC) == 0


def test_noalloc_entry_rejects_oversize_on_the_host():
    """ixh_gemv_noalloc refuses, before any GPU call, a request whose partial sums exceed its built-in buffer, and
    the atomic mode (which takes no workspace)."""
    lib = _lib.lib()
    s = _packed(out_f=1 << 14, in_f=1 << 14, bm0_words=1 << 23)
    assert lib.ixh_gemv_workspace_bytes(C.byref(s), 512, 16, 0) == 32 * 16 * (1 << 14) * 4 > (16 << 20)
    rc = lib.ixh_gemv_noalloc(C.byref(s), 0x1000, 512, 0x1000, 16, 1 << 14, 0x1000, 1 << 14, 0, None)
    assert rc == -4 and b"built-in buffer" in lib.ixh_last_error()
    rc = lib.ixh_gemv_noalloc(C.byref(s), 0x1000, 512, 0x1000, 1, 1 << 14, 0x1000, 1 << 14, _lib.IXH_GEMV_ATOMIC, None)
    assert rc == -1


@pytest.mark.parametrize("mutate,needle", [
    (lambda s: setattr(s, "n_levels", 1), "n_levels"),
    (lambda s: s.level_bits.__setitem__(2, 7), "last level"),
    (lambda s: s.level_bits.__setitem__(0, 6), "ascend"),
    (lambda s: setattr(s, "out_f", 1 << 20) or setattr(s, "in_f", 1 << 12), "31-bit"),
    (lambda s: s.bitmap_words.__setitem__(0, 0), "bitmap 0"),
    (lambda s: setattr(s, "scale", None), "scale"),
])
def test_malformed_packed_is_refused(mutate, needle):
    lib = _lib.lib()
    s = _packed()
    mutate(s)
    rc = lib.ixh_decode(C.byref(s), 0x1000, 8, None, 0x1000, None)
    assert rc == -1 and needle in lib.ixh_last_error().decode()


def test_malformed_gemv_arguments():
    lib = _lib.lib()
    s = _packed(out_f=4, in_f=1024, bm0_words=128)
    call = lambda chunk, m, x=0x1000, y=0x1000, ws=None, wsb=0, flags=0: lib.ixh_gemv(
        C.byref(s), 0x1000, chunk, x, m, 1024, y, 4, None, ws, wsb, flags, None)
    assert call(512, 0) == -1 and "m = 0" in lib.ixh_last_error().decode()
    assert call(512, 17) == -1
    assert call(500, 1) == -1 and "divide" in lib.ixh_last_error().decode()
    assert call(512, 1, x=None) == -1
    assert call(512, 1, y=None) == -1
    assert call(512, 1) == -4 and "workspace" in lib.ixh_last_error().decode()  # two chunks need partial sums
    assert call(512, 1, flags=_lib.IXH_GEMV_ATOMIC) == -1 and "y32" in lib.ixh_last_error().decode()
    with pytest.raises(_lib.IxhError):
        _lib.check(-1)


def test_malformed_encode_arguments():
    lib = _lib.lib()
    bits = (C.c_int32 * 3)(3, 5, 8)
    need = lib.ixh_encode_workspace_bytes(4, 1024, 3)
    assert need >= 1024 + 2 * 4  # 256 partial maxima and one tile sum for each of the two table rows
    assert lib.ixh_encode_workspace_bytes(0, 1024, 3) == 0 and lib.ixh_encode_workspace_bytes(4, 1024, 9) == 0
    scan = lambda out_f=4, in_f=1024, nl=3, lb=bits, w=0x1000, sc=0x1000, tab=0x1000, ws=0x1000, wsb=need: \
        lib.ixh_encode_scan(w, out_f, in_f, nl, lb, sc, tab, ws, wsb, None)
    assert scan(nl=1) == -1 and "n_levels" in lib.ixh_last_error().decode()
    assert scan(lb=(C.c_int32 * 3)(3, 5, 7)) == -1 and "last level" in lib.ixh_last_error().decode()
    assert scan(lb=(C.c_int32 * 3)(5, 3, 8)) == -1 and "ascend" in lib.ixh_last_error().decode()
    assert scan(out_f=0) == -1 and "empty" in lib.ixh_last_error().decode()
    assert scan(out_f=1 << 20, in_f=1 << 12) == -1 and "31-bit" in lib.ixh_last_error().decode()
    assert scan(w=None) == -1 and scan(sc=None) == -1 and scan(tab=None) == -1
    assert scan(wsb=need - 1) == -4 and "workspace" in lib.ixh_last_error().decode()
    s = _packed(out_f=4, in_f=1024, bm0_words=128)
    assert lib.ixh_encode_pack(None, C.byref(s), 0x1000, None) == -1
    assert lib.ixh_encode_pack(0x1000, C.byref(s), None, None) == -1
    s.bitmap_words[0] = 3
    assert lib.ixh_encode_pack(0x1000, C.byref(s), 0x1000, None) == -1 and "bitmap 0" in lib.ixh_last_error().decode()


def test_device_packed_refuses_cpu_tensors():
    from ixrun_amd.quantize import int8x_quantize

    p = int8x_quantize((torch.randn(8, 64) * 0.02).bfloat16())
    with pytest.raises(RuntimeError, match="GPU"):
        _lib.DevicePacked(p["level_bits"], 8, 64, p["bitmaps"], p["streams"], p["scale"].reshape(1))


def test_missing_library_is_loud(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libixhip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_bench_tables_are_well_formed():
    """bench.py's workload table (shape, rows, recipe[, level scheme]) and its table of measured HBM traffic, whose
    entries name sources that exist and workloads that the first table holds."""
    import os
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.path.insert(0, root)
    try:
        import bench
    finally:
        sys.path.remove(root)
    for name, spec in bench.WORKLOADS.items():
        assert len(spec) in (4, 5), name
        out_f, in_f, m, recipe = spec[:4]
        assert isinstance(out_f, int) and isinstance(in_f, int) and isinstance(m, int) and isinstance(recipe, str), name
        assert out_f > 0 and in_f > 0 and 0 <= m <= 512, name  # m = 0: decode and encode workloads
    for name, (nbytes, files, sha16) in bench.MEASURED_TRAFFIC_BYTES.items():
        assert nbytes > 0 and isinstance(sha16, str), name
        for f in files:
            assert os.path.exists(os.path.join(root, "ixrun_amd", "csrc", f)), (name, f)
