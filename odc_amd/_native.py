"""ctypes binding of libodc_hip.so (the C ABI declared in include/odc_hip.h).

This is the only place where Python touches the native library. It plays the part that
``odc/primitives/__init__.py:16-29`` plays in the reference (import the native extension, fail
hard when it has not been built): there is no Python or CPU fallback behind any entry point.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
import threading
from pathlib import Path

_PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = _PKG_DIR / "csrc"
INCLUDE_DIR = _PKG_DIR.parent / "include"
# $ODC_HIP_LIBRARY points at a library built elsewhere (same ABI); default: the in-tree build
LIB_PATH = Path(os.environ["ODC_HIP_LIBRARY"]) if os.environ.get("ODC_HIP_LIBRARY") else CSRC_DIR / "libodc_hip.so"
# host side (plain C++: arena, validation, launch planning) and device side (kernels, HIP runtime calls)
HOST_SOURCES = [CSRC_DIR / "odc_host.cpp"]
DEVICE_SOURCES = [CSRC_DIR / "odc_kernels.hip"]
SOURCES = HOST_SOURCES + DEVICE_SOURCES
# measurement-only companion: bare streaming kernels that bench.py times as the practical ceiling
CEILING_LIB_PATH = CSRC_DIR / "libodc_ceiling.so"
CEILING_SOURCES = [CSRC_DIR / "ceiling_kernels.hip"]

# every symbol include/odc_hip.h declares
EXPORTED_SYMBOLS = (
    "odc_arena_create",
    "odc_arena_destroy",
    "odc_arena_alloc",
    "odc_arena_free",
    "odc_arena_reset",
    "odc_arena_get_info",
    "odc_arena_ptr",
    "odc_arena_locate",
    "odc_gather",
    "odc_gather_cast",
    "odc_convert",
    "odc_scatter_accumulate",
    "odc_scatter_store",
    "odc_clear",
    "odc_publish",
    "odc_last_error",
    "odc_abi_version",
    "odc_set_option",
    "odc_get_option",
)

ABI_VERSION = 3
MAX_ITEMS_PER_LAUNCH = 64

ODC_OK = 0
ODC_ERR_INVALID = -1
ODC_ERR_NOMEM = -2
ODC_ERR_HIP = -3
ODC_ERR_UNSUPPORTED = -4
ODC_ERR_NOT_FOUND = -5
ODC_ERR_NO_BACKING = -6

ODC_ARENA_DEVICE = 0
ODC_ARENA_NO_BACKING = 1
ODC_ARENA_DRY_RUN = 2

DTYPE_BF16 = 0
DTYPE_F16 = 1
DTYPE_F32 = 2


class OdcNativeError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libodc_hip: {message} (status {code})")
        self.code = code
        self.message = message


class ArenaInfo(ctypes.Structure):
    _fields_ = [
        ("world_size", ctypes.c_uint32),
        ("device", ctypes.c_int32),
        ("flags", ctypes.c_uint32),
        ("n_allocations", ctypes.c_uint32),
        ("bytes_per_rank", ctypes.c_uint64),
        ("rank_stride", ctypes.c_uint64),
        ("base", ctypes.c_uint64),
        ("bytes_in_use", ctypes.c_uint64),
        ("high_water", ctypes.c_uint64),
    ]


class GatherItem(ctypes.Structure):
    _fields_ = [
        ("dst", ctypes.c_void_p),
        ("src_offset", ctypes.c_uint64),
        ("shard_bytes", ctypes.c_uint64),
    ]


class AccumItem(ctypes.Structure):
    _fields_ = [
        ("grad", ctypes.c_void_p),
        ("grad_elems", ctypes.c_uint64),
        ("acc_offset", ctypes.c_uint64),
        ("shard_elems", ctypes.c_uint64),
    ]


class GatherCastItem(ctypes.Structure):
    _fields_ = [
        ("dst", ctypes.c_void_p),
        ("src_offset", ctypes.c_uint64),
        ("shard_elems", ctypes.c_uint64),
    ]


class ConvertItem(ctypes.Structure):
    _fields_ = [
        ("src_offset", ctypes.c_uint64),
        ("dst_offset", ctypes.c_uint64),
        ("elems", ctypes.c_uint64),
    ]


class PublishItem(ctypes.Structure):
    _fields_ = [
        ("acc_offset", ctypes.c_uint64),
        ("elems", ctypes.c_uint64),
        ("out", ctypes.c_void_p),
    ]


class Span(ctypes.Structure):
    _fields_ = [("offset", ctypes.c_uint64), ("nbytes", ctypes.c_uint64)]


def hipcc_command(output: Path = LIB_PATH, sources=None) -> list[str]:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    return [
        hipcc,
        "-O3",
        "-std=c++17",
        "--offload-arch=gfx950",
        # keep hipcc from fusing float pairs into packed-fp32 instructions
        "-Xclang",
        "-target-feature",
        "-Xclang",
        "-packed-fp32-ops",
        "-fPIC",
        "-shared",
        f"-I{INCLUDE_DIR}",
        f"-I{CSRC_DIR}",
        "-o",
        str(output),
        *_with_languages(SOURCES if sources is None else sources),
    ]


def _with_languages(sources) -> list[str]:
    """hipcc arguments for a mixed list: .cpp files are plain C++ (host only), .hip files HIP."""
    args = []
    for src in sources:
        args += ["-x", "hip" if str(src).endswith(".hip") else "c++", str(src)]
    return args


def _run_hipcc(cmd, verbose: bool) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or proc.returncode != 0:
        print(" ".join(cmd))
        print(proc.stdout)
        print(proc.stderr)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {proc.returncode}")


def build_library(verbose: bool = False) -> Path:
    """Compile libodc_hip.so in-tree for gfx950 (works without a GPU)."""
    _run_hipcc(hipcc_command(), verbose)
    return LIB_PATH


def build_ceiling_library(verbose: bool = False) -> Path:
    """Compile libodc_ceiling.so (bench.py's bare streaming kernels) in-tree for gfx950."""
    _run_hipcc(hipcc_command(CEILING_LIB_PATH, CEILING_SOURCES), verbose)
    return CEILING_LIB_PATH


def load_ceiling() -> ctypes.CDLL:
    """The measurement-only ceiling kernels; built on first use when missing."""
    if not CEILING_LIB_PATH.exists():
        build_ceiling_library()
    lib = ctypes.CDLL(str(CEILING_LIB_PATH))
    vp, u64, u32, ci = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int
    P = ctypes.POINTER
    lib.odc_ceiling_read.argtypes = [vp, u64, vp, ci, u32, vp, P(u64)]
    lib.odc_ceiling_write.argtypes = [vp, u64, ci, u32, vp, P(u64)]
    lib.odc_ceiling_copy.argtypes = [vp, vp, u64, ci, u32, vp, P(u64)]
    lib.odc_ceiling_rmw.argtypes = [vp, vp, u64, ci, u32, vp, P(u64)]
    lib.odc_ceiling_set_threads.argtypes = [ci]
    for name in ("odc_ceiling_read", "odc_ceiling_write", "odc_ceiling_copy", "odc_ceiling_rmw",
                 "odc_ceiling_set_threads"):
        getattr(lib, name).restype = ci
    return lib


_lib = None
_lib_lock = threading.Lock()


def _declare(lib: ctypes.CDLL) -> None:
    vp, u32, u64, i64, ci = (
        ctypes.c_void_p,
        ctypes.c_uint32,
        ctypes.c_uint64,
        ctypes.c_int64,
        ctypes.c_int,
    )
    P = ctypes.POINTER
    lib.odc_arena_create.argtypes = [u32, u64, u32, P(vp)]
    lib.odc_arena_destroy.argtypes = [vp]
    lib.odc_arena_alloc.argtypes = [vp, u64, P(u64)]
    lib.odc_arena_free.argtypes = [vp, u64]
    lib.odc_arena_reset.argtypes = [vp]
    lib.odc_arena_get_info.argtypes = [vp, P(ArenaInfo)]
    lib.odc_arena_ptr.argtypes = [vp, u32, u64]
    lib.odc_arena_ptr.restype = vp
    lib.odc_arena_locate.argtypes = [vp, vp, P(u32), P(u64), P(u64)]
    lib.odc_gather.argtypes = [vp, P(GatherItem), u32, u32, vp]
    lib.odc_gather_cast.argtypes = [vp, P(GatherCastItem), u32, ci, ci, u32, vp]
    lib.odc_convert.argtypes = [vp, P(ConvertItem), u32, ci, ci, vp]
    lib.odc_scatter_accumulate.argtypes = [vp, P(AccumItem), u32, ci, ci, vp]
    lib.odc_scatter_store.argtypes = [vp, P(AccumItem), u32, ci, ci, vp]
    lib.odc_publish.argtypes = [vp, u32, P(PublishItem), u32, ci, ci, ctypes.c_float, vp]
    lib.odc_clear.argtypes = [vp, P(Span), u32, vp]
    lib.odc_last_error.argtypes = []
    lib.odc_last_error.restype = ctypes.c_char_p
    lib.odc_abi_version.argtypes = []
    lib.odc_set_option.argtypes = [ctypes.c_char_p, i64]
    lib.odc_get_option.argtypes = [ctypes.c_char_p, P(i64)]
    for name in EXPORTED_SYMBOLS:
        fn = getattr(lib, name)
        if name not in ("odc_arena_ptr", "odc_last_error"):
            fn.restype = ci


def load() -> ctypes.CDLL:
    """Load the in-tree library; raise if it is missing or has the wrong ABI."""
    global _lib
    with _lib_lock:
        if _lib is None:
            if not LIB_PATH.exists():
                # nothing built yet: build once, in-tree; there is no fallback path
                try:
                    build_library()
                except (OSError, RuntimeError) as e:
                    raise ImportError(
                        f"{LIB_PATH} is missing and could not be built ({e}): run "
                        "`python -c 'import __graft_entry__ as g; g.build()'` (needs hipcc)"
                    ) from None
            # torch ships a HIP runtime of its own and must load it before this library pulls in
            # the system's by name: two HIP runtimes in one process do not both see the device
            # (a program that imported this package before torch found "no ROCm-capable device")
            import torch  # noqa: F401

            lib = ctypes.CDLL(str(LIB_PATH))
            try:
                _declare(lib)
            except AttributeError as e:
                raise ImportError(f"{LIB_PATH} is stale ({e}): rebuild it") from None
            got = lib.odc_abi_version()
            if got != ABI_VERSION:
                raise ImportError(f"{LIB_PATH} has ABI version {got}, expected {ABI_VERSION}: rebuild it")
            _lib = lib
    return _lib


def check(status: int) -> None:
    if status != ODC_OK:
        raise OdcNativeError(status, load().odc_last_error().decode("utf-8", "replace"))


def set_option(name: str, value: int) -> None:
    check(load().odc_set_option(name.encode(), int(value)))


def get_option(name: str) -> int:
    out = ctypes.c_int64(0)
    check(load().odc_get_option(name.encode(), ctypes.byref(out)))
    return out.value
