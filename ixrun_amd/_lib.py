"""ctypes binding of ``libixhip.so`` (the C ABI declared in ``include/ixhip.h``; the testing hook in
``include/ixhip_test.h``).

The library is built in-tree by ``csrc/build.sh``.  There is no CPU fallback:
if the shared object is missing, or a call is made without a GPU tensor,
loading or the call raises.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# IXH_LIB names another build of the library (development); the default is the in-tree one
LIB_PATH = os.environ.get("IXH_LIB") or os.path.join(_HERE, "csrc", "libixhip.so")

IXH_MAX_LEVELS = 8
IXH_GEMV_ATOMIC = 1
IXH_GEMV_FORCE_GENERIC = 2
IXH_GEMV_COLUMN_KERNEL = 4
IXH_GEMV_FORCE_358 = 8
IXH_GEMV_STAGED = 16
IXH_GEMV_DENSE = 32

IXH_EUNSUPPORTED = -2
ERROR_NAMES = {-1: "IXH_EINVAL", -2: "IXH_EUNSUPPORTED", -3: "IXH_ELAUNCH", -4: "IXH_EWORKSPACE"}


class IxhPacked(C.Structure):
    _fields_ = [
        ("n_levels", C.c_int32),
        ("level_bits", C.c_int32 * IXH_MAX_LEVELS),
        ("out_f", C.c_int64),
        ("in_f", C.c_int64),
        ("bitmaps", C.c_void_p * (IXH_MAX_LEVELS - 1)),
        ("bitmap_words", C.c_uint64 * (IXH_MAX_LEVELS - 1)),
        ("streams", C.c_void_p * (IXH_MAX_LEVELS - 1)),
        ("stream_words", C.c_uint64 * (IXH_MAX_LEVELS - 1)),
        ("last", C.c_void_p),
        ("last_bytes", C.c_uint64),
        ("scale", C.c_void_p),
    ]


class IxhError(RuntimeError):
    """A call into libixhip returned a negative code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"{ERROR_NAMES.get(code, code)}: {message}")
        self.code = code


_lib = None

# the product interface (include/ixhip.h) and the testing hook (include/ixhip_test.h)
EXPORTS = (
    "ixh_version", "ixh_last_error", "ixh_prefix_entries", "ixh_prefix_build", "ixh_decode",
    "ixh_gemv", "ixh_gemv_workspace_bytes", "ixh_gemv_noalloc", "ixh_gemm", "ixh_gemm_workspace_bytes",
    "ixh_encode_workspace_bytes", "ixh_encode_scan", "ixh_encode_pack", "ixh_decode_gs",
)
TEST_EXPORTS = ("ixh_set_option",)


def lib() -> C.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with ixrun_amd/csrc/build.sh "
                "(hipcc --offload-arch=gfx950); there is no fallback path"
            )
        L = C.CDLL(LIB_PATH)
        L.ixh_version.restype = C.c_int
        L.ixh_last_error.restype = C.c_char_p
        L.ixh_set_option.restype = C.c_int
        L.ixh_set_option.argtypes = [C.c_char_p, C.c_int64]
        L.ixh_prefix_entries.restype = C.c_int64
        L.ixh_prefix_entries.argtypes = [C.c_int64, C.c_int64]
        L.ixh_prefix_build.restype = C.c_int
        L.ixh_prefix_build.argtypes = [C.POINTER(IxhPacked), C.c_int64, C.c_void_p, C.c_void_p]
        L.ixh_decode.restype = C.c_int
        L.ixh_decode.argtypes = [C.POINTER(IxhPacked), C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]
        L.ixh_decode_gs.restype = C.c_int
        L.ixh_decode_gs.argtypes = [C.POINTER(IxhPacked), C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p,
                                    C.c_void_p]
        L.ixh_gemv.restype = C.c_int
        L.ixh_gemv.argtypes = [
            C.POINTER(IxhPacked), C.c_void_p, C.c_int64, C.c_void_p, C.c_int32, C.c_int64, C.c_void_p,
            C.c_int64, C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint32, C.c_void_p,
        ]
        L.ixh_gemv_noalloc.restype = C.c_int
        L.ixh_gemv_noalloc.argtypes = [
            C.POINTER(IxhPacked), C.c_void_p, C.c_int64, C.c_void_p, C.c_int32, C.c_int64, C.c_void_p,
            C.c_int64, C.c_uint32, C.c_void_p,
        ]
        L.ixh_gemv_workspace_bytes.restype = C.c_size_t
        L.ixh_gemv_workspace_bytes.argtypes = [C.POINTER(IxhPacked), C.c_int64, C.c_int32, C.c_uint32]
        L.ixh_gemm.restype = C.c_int
        L.ixh_gemm.argtypes = [
            C.POINTER(IxhPacked), C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_void_p, C.c_int64,
            C.c_void_p, C.c_size_t, C.c_void_p,
        ]
        L.ixh_gemm_workspace_bytes.restype = C.c_size_t
        L.ixh_gemm_workspace_bytes.argtypes = [C.POINTER(IxhPacked), C.c_int32]
        L.ixh_encode_workspace_bytes.restype = C.c_size_t
        L.ixh_encode_workspace_bytes.argtypes = [C.c_int64, C.c_int64, C.c_int32]
        L.ixh_encode_scan.restype = C.c_int
        L.ixh_encode_scan.argtypes = [
            C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.POINTER(C.c_int32), C.c_void_p, C.c_void_p,
            C.c_void_p, C.c_size_t, C.c_void_p,
        ]
        L.ixh_encode_pack.restype = C.c_int
        L.ixh_encode_pack.argtypes = [C.c_void_p, C.POINTER(IxhPacked), C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def check(code: int) -> None:
    if code != 0:
        raise IxhError(code, lib().ixh_last_error().decode())


DECODE_KERNELS = {"auto": 0, "rows": 1, "dense": 2, "staged": 3, "generic": 4}


def set_option(name: str, value) -> None:
    """Process-wide testing / measurement switch of the library (``ixh_set_option``, declared in
    ``include/ixhip_test.h``, not in the product header); ``decode_kernel`` also takes the decoder's name."""
    if name == "decode_kernel" and isinstance(value, str):
        value = DECODE_KERNELS[value]
    check(lib().ixh_set_option(name.encode(), int(value)))


def current_stream(device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_cuda(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{what} must live on the GPU (got {t.device}); the HIP path has no CPU fallback")
    if not t.is_contiguous():
        raise RuntimeError(f"{what} must be contiguous")


class DevicePacked:
    """An ``IxhPacked`` built over device tensors that it keeps alive."""

    def __init__(self, level_bits, out_f, in_f, bitmaps, streams, scale):
        level_bits = tuple(int(b) for b in level_bits)
        n_levels = len(level_bits)
        if not 2 <= n_levels <= IXH_MAX_LEVELS:
            raise ValueError(f"{n_levels} levels: the device path takes 2..{IXH_MAX_LEVELS}")
        if len(bitmaps) != n_levels - 1 or len(streams) != n_levels:
            raise ValueError("need one bitmap per level but the last and one stream per level")
        self.level_bits, self.out_f, self.in_f = level_bits, int(out_f), int(in_f)
        self.N = self.out_f * self.in_f
        # scale None: the group-scale format, whose scales are an argument of its decode call
        self.tensors = list(bitmaps) + list(streams) + ([scale] if scale is not None else [])
        for i, t in enumerate(self.tensors):
            _require_cuda(t, f"packed tensor {i}")
        if scale is not None and (scale.dtype != torch.bfloat16 or scale.numel() != 1):
            raise ValueError("scale must be a one-element bf16 tensor")
        self.device = self.tensors[0].device
        s = IxhPacked()
        s.n_levels = n_levels
        for i, b in enumerate(level_bits):
            s.level_bits[i] = b
        s.out_f, s.in_f = self.out_f, self.in_f
        for i in range(n_levels - 1):
            bm, st = bitmaps[i], streams[i]
            if bm.dtype != torch.int32 or st.dtype != torch.int32:
                raise ValueError("bitmaps and packed streams must be torch.int32")
            s.bitmaps[i] = bm.data_ptr() if bm.numel() else None
            s.bitmap_words[i] = bm.numel()
            s.streams[i] = st.data_ptr() if st.numel() else None
            s.stream_words[i] = st.numel()
        last = streams[-1]
        if last.dtype != torch.uint8:
            raise ValueError("the last stream must be torch.uint8")
        s.last = last.data_ptr() if last.numel() else None
        s.last_bytes = last.numel()
        s.scale = scale.data_ptr() if scale is not None else None
        self.struct = s

    @classmethod
    def from_dict(cls, packed: dict, device=None) -> "DevicePacked":
        dev = torch.device(device if device is not None else "cuda")
        mv = lambda t: t.to(dev).contiguous()
        return cls(packed["level_bits"], packed["out_f"], packed["in_f"],
                   [mv(b) for b in packed["bitmaps"]], [mv(s) for s in packed["streams"]],
                   mv(packed["scale"].reshape(1)))

    # ---- thin call wrappers -------------------------------------------------
    def prefix_entries(self, chunk: int) -> int:
        return int(lib().ixh_prefix_entries(self.N, int(chunk)))

    def prefix_build(self, chunk: int) -> torch.Tensor:
        """int32 [n_levels-1, entries] rank table at flat positions u*chunk (device)."""
        entries = self.prefix_entries(chunk)
        if entries < 1:
            raise ValueError(f"chunk {chunk} must be positive")
        table = torch.empty((len(self.level_bits) - 1, entries), dtype=torch.int32, device=self.device)
        check(lib().ixh_prefix_build(C.byref(self.struct), int(chunk), table.data_ptr(), current_stream(self.device)))
        return table

    def decode(self, table: torch.Tensor, chunk: int, out_i8=None, out_bf16=None) -> None:
        for t, dt in ((out_i8, torch.int8), (out_bf16, torch.bfloat16)):
            if t is not None:
                _require_cuda(t, "decode output")
                if t.dtype != dt or t.numel() < self.N:
                    raise ValueError(f"decode output must be {dt} with at least {self.N} elements")
        check(lib().ixh_decode(
            C.byref(self.struct), table.data_ptr(), int(chunk),
            out_i8.data_ptr() if out_i8 is not None else None,
            out_bf16.data_ptr() if out_bf16 is not None else None, current_stream(self.device)))

    def decode_gs(self, table: torch.Tensor, chunk: int, group_scales: torch.Tensor, group_size: int,
                  out_bf16: torch.Tensor) -> None:
        """Decode with one fp16 scale per `group_size` consecutive elements (the group-scale format)."""
        _require_cuda(group_scales, "group_scales")
        _require_cuda(out_bf16, "decode output")
        n_groups = -(-self.N // int(group_size)) if int(group_size) > 0 else 0  # the library rejects sizes <= 0
        if group_scales.dtype != torch.float16 or group_scales.numel() < n_groups:
            raise ValueError(f"group_scales must be fp16 with at least {n_groups} elements")
        if out_bf16.dtype != torch.bfloat16 or out_bf16.numel() < self.N:
            raise ValueError(f"decode output must be bf16 with at least {self.N} elements")
        check(lib().ixh_decode_gs(C.byref(self.struct), table.data_ptr(), int(chunk), group_scales.data_ptr(),
                                  int(group_size), out_bf16.data_ptr(), current_stream(self.device)))

    def gemv_workspace_bytes(self, chunk: int, m: int, flags: int = 0) -> int:
        return int(lib().ixh_gemv_workspace_bytes(C.byref(self.struct), int(chunk), int(m), int(flags)))

    def _gemv_operands(self, table, chunk, x, y, y32, workspace):
        """Check every buffer of a fused call on the host (device, dtype, layout, size): the kernels trust the
        pointers they are given.  Returns (x as [M, in_f], M, ldx, ldy)."""
        if not x.is_cuda:
            raise RuntimeError(f"x must live on the GPU (got {x.device}); the HIP path has no CPU fallback")
        if x.dtype != torch.bfloat16:
            raise ValueError("x must be bf16")
        x2 = x.reshape(-1, self.in_f)
        if x2.stride(1) != 1:
            raise ValueError("x rows must be contiguous")
        m = x2.shape[0]
        ldx = x2.stride(0) if m > 1 else self.in_f
        ldy = self.out_f
        for name, t, dt in (("y", y, torch.bfloat16), ("y32", y32, torch.float32)):
            if t is None:
                continue
            if not t.is_cuda or t.device != self.device:
                raise RuntimeError(f"{name} must live on {self.device} (got {t.device})")
            if t.dtype != dt:
                raise ValueError(f"{name} must be {dt}")
            if name == "y" and t.dim() == 2 and m > 1:  # rows may be strided (ldy); y32 is always dense [M, out_f]
                if t.shape[0] < m or t.shape[1] < self.out_f or t.stride(1) != 1 or t.stride(0) < self.out_f:
                    raise ValueError(f"y must hold {m} contiguous rows of {self.out_f} elements")
                ldy = t.stride(0)
            elif not t.is_contiguous() or t.numel() < m * self.out_f:
                raise ValueError(f"{name} must be contiguous with at least {m * self.out_f} elements")
        entries = self.prefix_entries(chunk)
        if entries < 1:
            raise ValueError(f"chunk {chunk} must be positive")
        if not table.is_cuda or table.device != self.device:
            raise RuntimeError(f"the rank table must live on {self.device} (got {table.device})")
        if (table.dtype != torch.int32 or table.dim() != 2 or table.shape[0] < len(self.level_bits) - 1
                or table.shape[1] != entries or table.stride(1) != 1 or table.stride(0) != entries):
            raise ValueError(f"the rank table must be contiguous int32 [{len(self.level_bits) - 1}, {entries}] "
                             f"for chunk {chunk}")
        if workspace is not None:
            if not workspace.is_cuda or workspace.device != self.device:
                raise RuntimeError(f"the workspace must live on {self.device} (got {workspace.device})")
            if not workspace.is_contiguous():
                raise ValueError("the workspace must be contiguous")
        return x2, m, ldx, ldy

    def gemv(self, table, chunk, x, y=None, y32=None, workspace=None, flags=0) -> None:
        """x bf16 [M, in_f] (row stride x.stride(0)); y bf16 [M, out_f] or y32 fp32 (atomic mode)."""
        x2, m, ldx, ldy = self._gemv_operands(table, chunk, x, y, y32, workspace)
        check(lib().ixh_gemv(
            C.byref(self.struct), table.data_ptr(), int(chunk), x2.data_ptr(), m, ldx,
            y.data_ptr() if y is not None else None, ldy,
            y32.data_ptr() if y32 is not None else None,
            workspace.data_ptr() if workspace is not None else None,
            workspace.numel() * workspace.element_size() if workspace is not None else 0,
            int(flags), current_stream(self.device)))

    def gemv_noalloc(self, table, chunk, x, y, flags=0) -> None:
        """``gemv`` through the entry point that allocates nothing: partial sums go to the library's own buffer
        (``IXH_NOALLOC_WORKSPACE_BYTES``); requests whose kernel cannot fit its partial sums there raise
        ``IxhError(IXH_EWORKSPACE)``."""
        if y is None:
            raise ValueError("gemv_noalloc needs the bf16 output y")
        x2, m, ldx, ldy = self._gemv_operands(table, chunk, x, y, None, None)
        with torch.cuda.device(self.device):
            check(lib().ixh_gemv_noalloc(
                C.byref(self.struct), table.data_ptr(), int(chunk), x2.data_ptr(), m, ldx, y.data_ptr(), ldy,
                int(flags), current_stream(self.device)))

    def gemm_workspace_bytes(self, m: int) -> int:
        return int(lib().ixh_gemm_workspace_bytes(C.byref(self.struct), int(m)))

    def gemm(self, table512, x, y, workspace) -> None:
        """Fused decode + matrix-core GEMM: x bf16 [M, in_f], y bf16 [M, out_f], any M; table512 is the
        rank table at unit 512.  Raises IxhError(IXH_EUNSUPPORTED) for shapes the kernel does not take."""
        if not x.is_cuda:
            raise RuntimeError(f"x must live on the GPU (got {x.device}); the HIP path has no CPU fallback")
        if x.dtype != torch.bfloat16 or y.dtype != torch.bfloat16:
            raise ValueError("x and y must be bf16")
        x2 = x.reshape(-1, self.in_f)
        if x2.stride(1) != 1 or y.stride(-1) != 1:
            raise ValueError("x and y rows must be contiguous")
        m = x2.shape[0]
        y2 = y.reshape(m, self.out_f)
        check(lib().ixh_gemm(
            C.byref(self.struct), table512.data_ptr(), x2.data_ptr(), m,
            x2.stride(0) if m > 1 else self.in_f, y2.data_ptr(), y2.stride(0) if m > 1 else self.out_f,
            workspace.data_ptr() if workspace is not None else None,
            workspace.numel() * workspace.element_size() if workspace is not None else 0,
            current_stream(self.device)))


def encode_device(weight: torch.Tensor, level_bits) -> tuple:
    """Encode a bf16 [out_f, in_f] device tensor with the library's two encoder calls.

    Returns ``(DevicePacked, table512, counts)``: the packed tensors (device), the int32
    ``[n_levels-1, entries]`` rank table at unit 512 and the per-level element counts (host ints).  One
    host synchronisation (reading the counts) sits between the two calls.
    """
    _require_cuda(weight, "weight")
    if weight.dtype != torch.bfloat16 or weight.dim() != 2:
        raise ValueError("the device encoder takes a 2-D bf16 weight")
    level_bits = tuple(int(b) for b in level_bits)
    n_levels = len(level_bits)
    out_f, in_f = weight.shape
    dev = weight.device
    L = lib()
    bits = (C.c_int32 * n_levels)(*level_bits)
    entries = int(L.ixh_prefix_entries(out_f * in_f, 512))
    ws_bytes = int(L.ixh_encode_workspace_bytes(out_f, in_f, n_levels))
    workspace = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
    scale = torch.empty(1, dtype=torch.bfloat16, device=dev)
    table = torch.empty((max(n_levels - 1, 1), max(entries, 1)), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        check(L.ixh_encode_scan(weight.data_ptr(), out_f, in_f, n_levels, bits, scale.data_ptr(), table.data_ptr(),
                                workspace.data_ptr(), ws_bytes, current_stream(dev)))
        counts = [int(c) for c in table[:, -1].cpu().tolist()]  # the one synchronisation
        counts.append(out_f * in_f - sum(counts))
        left = out_f * in_f
        bitmaps, streams = [], []
        for i, b in enumerate(level_bits[:-1]):
            bitmaps.append(torch.empty((left + 31) // 32, dtype=torch.int32, device=dev))
            streams.append(torch.empty((counts[i] * b + 31) // 32, dtype=torch.int32, device=dev))
            left -= counts[i]
        streams.append(torch.empty(counts[-1], dtype=torch.uint8, device=dev))
        dp = DevicePacked(level_bits, out_f, in_f, bitmaps, streams, scale)
        check(L.ixh_encode_pack(weight.data_ptr(), C.byref(dp.struct), table.data_ptr(), current_stream(dev)))
    return dp, table, counts
