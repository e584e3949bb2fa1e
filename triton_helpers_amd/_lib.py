"""ctypes binding of ``libnf_cdna4.so`` (declared in ``include/nf_cdna4.h``).

The library is the only compute path: if it is missing or fails to load, every
operator of this package raises instead of falling back to anything else.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p
from pathlib import Path
from typing import Optional

import torch

LIB_PATH = Path(__file__).resolve().parent / "libnf_cdna4.so"

NF_ABI_VERSION = 9
NF_F32, NF_F16, NF_BF16 = 0, 1, 2
NF_ACT = {"none": 0, "relu": 1, "silu": 2, "relu2": 3, "gelu": 4}
NF_MAX_LEVELS = 32
NF_MAX_DIMS = 6
NF_EINVAL, NF_EUNSUPPORTED, NF_EALIGN = -1, -2, -3
NF_HASH_FORCE_GENERIC = 1
NF_HASH_FORCE_ATOMIC = 2
NF_HASH_FORCE_PLANES = 4
NF_HASH_FWD_STAGED = 8
NF_HASH_BWD_RECORDS = 16
NF_ADAM_CLEAR_GRAD, NF_ADAM_SKIP_NONFINITE = 1, 2

_DTYPE_CODE = {torch.float32: NF_F32, torch.float16: NF_F16, torch.bfloat16: NF_BF16}

EXPORTS = (
    "nf_abi_version",
    "nf_last_error",
    "nf_hash_encode_fwd",
    "nf_hash_encode_bwd",
    "nf_hash_encode_bwd_workspace_bytes",
    "nf_hash_encode_bwd_static",
    "nf_hash_encode_bwd_static_bytes",
    "nf_hash_encode_indices",
    "nf_hash_encode_indices_fast",
    "nf_hash_check_host",
    "nf_table_adam_step",
    "nf_mlp_fwd",
    "nf_mlp_bwd",
    "nf_mlp_workspace_bytes",
    "nf_mlp_bwd_rounded",
    "nf_mlp_bwd_rounded_workspace_bytes",
    "nf_revmlp_fwd",
    "nf_revmlp_bwd",
)


class HashGeom(Structure):
    """Mirror of ``nf_hash_geom``."""

    _fields_ = [
        ("dims", c_int32),
        ("feat", c_int32),
        ("levels", c_int32),
        ("first_hash_level", c_int32),
        ("max_rows", c_int64),
        ("res", c_int32 * NF_MAX_LEVELS),
        ("rows", c_int64 * NF_MAX_LEVELS),
        ("row_offset", c_int64 * NF_MAX_LEVELS),
    ]


class NativeLibraryError(RuntimeError):
    pass


_lib: Optional[ctypes.CDLL] = None


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}; expected float32, float16 or bfloat16") from None


def _declare(lib: ctypes.CDLL) -> None:
    P, I64, I = c_void_p, c_int64, c_int
    lib.nf_abi_version.restype = c_int
    lib.nf_abi_version.argtypes = []
    lib.nf_last_error.restype = c_char_p
    lib.nf_last_error.argtypes = []
    lib.nf_hash_encode_fwd.restype = c_int
    lib.nf_hash_encode_fwd.argtypes = [P, I, I64, I64, P, I, P, I64, I64, POINTER(HashGeom), P, c_float, I, P]
    lib.nf_hash_encode_bwd.restype = c_int
    lib.nf_hash_encode_bwd.argtypes = [P, I, I64, I64, P, I, I64, P, I64, POINTER(HashGeom), P, c_float, P, I64, I, P]
    lib.nf_hash_encode_bwd_workspace_bytes.restype = c_int64
    lib.nf_hash_encode_bwd_workspace_bytes.argtypes = [I64, POINTER(HashGeom), I, I]
    lib.nf_hash_encode_bwd_static.restype = c_int
    lib.nf_hash_encode_bwd_static.argtypes = [P, I, I64, I64, P, I, I64, P, I64, POINTER(HashGeom), P, c_float, I, P]
    lib.nf_hash_encode_bwd_static_bytes.restype = c_int64
    lib.nf_hash_encode_bwd_static_bytes.argtypes = []
    lib.nf_hash_encode_indices.restype = c_int
    lib.nf_hash_encode_indices.argtypes = [P, I, I64, I64, P, P, I64, POINTER(HashGeom), P, c_float, P]
    lib.nf_hash_encode_indices_fast.restype = c_int
    lib.nf_hash_encode_indices_fast.argtypes = [P, I, I64, I64, P, P, I64, POINTER(HashGeom), P, c_float, P]
    lib.nf_hash_check_host.restype = c_int
    lib.nf_hash_check_host.argtypes = [P, I64, POINTER(HashGeom), P, c_float, I, P, P, P]
    lib.nf_table_adam_step.restype = c_int
    lib.nf_table_adam_step.argtypes = [P, I, P, P, P, P, I64, I64, c_float, c_float, c_float, c_float, c_float, c_float, I, P, P]
    lib.nf_mlp_fwd.restype = c_int
    lib.nf_mlp_fwd.argtypes = [P, I64, P, I64, P, P, P, P, P, P, I64, I, I, I, I, I, I, I, P, I64, P]
    lib.nf_mlp_bwd_rounded.restype = c_int
    lib.nf_mlp_bwd_rounded.argtypes = [P, I64, P, I64, P, I64, P, P, P, P, P, P, P, P, P, P, P, P, I64, I, I, I, I, I, I, I, P, I64, P]
    lib.nf_mlp_bwd_rounded_workspace_bytes.restype = I64
    lib.nf_mlp_bwd_rounded_workspace_bytes.argtypes = [I, I, I]
    lib.nf_mlp_workspace_bytes.restype = I64
    lib.nf_mlp_workspace_bytes.argtypes = [I64, I, I, I, I, I]
    lib.nf_mlp_bwd.restype = c_int
    lib.nf_mlp_bwd.argtypes = [P, I64, P, I64, P, I64, P, P, P, P, P, P, P, P, P, P, P, P, I64, I, I, I, I, I, I, I, P, I64, P]
    lib.nf_revmlp_fwd.restype = c_int
    lib.nf_revmlp_fwd.argtypes = [P, I64, P, I64, P, P, P, P, I64, I, I, I, I, P]
    lib.nf_revmlp_bwd.restype = c_int
    lib.nf_revmlp_bwd.argtypes = [P, I64, P, I64, P, I64, P, I64, P, P, P, P, P, P, P, P, I64, I, I, I, I, P]


def load() -> ctypes.CDLL:
    """Load (once) and return the native library; raises ``NativeLibraryError`` if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise NativeLibraryError(
            f"{LIB_PATH} is missing: build it with `python -m triton_helpers_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no fallback path."
        )
    try:
        lib = ctypes.CDLL(str(LIB_PATH))
    except OSError as e:
        raise NativeLibraryError(f"cannot load {LIB_PATH}: {e}") from e
    missing = [n for n in EXPORTS if not hasattr(lib, n)]
    if missing:
        raise NativeLibraryError(f"{LIB_PATH} lacks symbols {missing}")
    _declare(lib)
    if lib.nf_abi_version() != NF_ABI_VERSION:
        raise NativeLibraryError(f"ABI version {lib.nf_abi_version()} != expected {NF_ABI_VERSION}; rebuild the library")
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    """Turn a non-zero return code of the library into ``RuntimeError``."""
    if rc != 0:
        msg = load().nf_last_error()
        raise RuntimeError(f"{what} failed (code {rc}): {msg.decode() if msg else ''}")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device: torch.device) -> int:
    """Handle of the current stream of ``device`` (the raw accessor saves the Stream object, two microseconds a call)."""
    if _raw_stream is not None:
        index = device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream


class GradBuffers:
    """float32 zero accumulators shaped like the given tensors (``None`` stays ``None``), carved out of one buffer
    so that a single fill kernel clears them all and a single cast kernel rounds them all to the parameters' dtype.
    The kernels only need addresses, so no view tensors are made for the accumulators (each tensor op costs the host
    a few microseconds, which is what bounds a small step)."""

    def __init__(self, *tensors):
        self._like = tensors
        self._offsets, off = [], 0
        for t in tensors:
            self._offsets.append(off)
            if t is not None:
                off += (t.numel() + 3) // 4 * 4  # 16-byte aligned pieces
        self.flat = torch.zeros(off, dtype=torch.float32, device=next(t for t in tensors if t is not None).device) if off else None

    def pointers(self):
        """Device addresses of the accumulators (``None`` where the tensor is absent)."""
        base = self.flat.data_ptr() if self.flat is not None else 0
        return tuple(None if t is None else base + 4 * o for t, o in zip(self._like, self._offsets))

    def rounded(self, dtype):
        """The accumulators rounded once to ``dtype`` (what autograd would do tensor by tensor), as views."""
        if self.flat is None:
            return tuple(None for _ in self._like)
        flat = self.flat if dtype == torch.float32 else self.flat.to(dtype)
        return tuple(None if t is None else flat.as_strided(t.shape, t.stride(), o) if t.is_contiguous()
                     else flat[o:o + t.numel()].view(t.shape) for t, o in zip(self._like, self._offsets))
