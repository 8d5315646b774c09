"""ctypes binding of ``libartab_attention.so`` (the C ABI in ``include/artab_attention.h``).

There is no CPU fallback: if the shared library has not been built the first use
raises ``RuntimeError`` naming the build command, and tensors that are not on a
HIP device are rejected.

``libartab_bench.so`` (``include/artab_bench.h``) is a second link of the same object files with
the benchmark aids added; ``benchmark_library()`` routes every call of this package through it for
the duration of a ``with`` block.  Only ``bench.py`` does that.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libartab_attention.so")
BENCH_LIB_PATH = os.path.join(_HERE, "libartab_bench.so")

ABI_VERSION = 7  # ARTAB_VERSION of include/artab_attention.h
STATIC_SCRATCH_BYTES = 32 << 20  # ARTAB_STATIC_SCRATCH_BYTES
ARTAB_BF16, ARTAB_F16, ARTAB_F32 = 0, 1, 2
IMPL_AUTO, IMPL_PORTABLE, IMPL_MFMA = 0, 1, 2

ORDER_WAIT = 1            # artab_attention_partials.order_flags
ORDER_CONSUMER_WAITS = 2  # flags of artab_decode_attention_partials_ordered
ARTAB_ERR_NULL_POINTER = -1
ARTAB_ERR_BAD_SHAPE = -2
ARTAB_ERR_BAD_STRIDE = -3
ARTAB_ERR_UNSUPPORTED = -4
ARTAB_ERR_WORKSPACE = -5
ARTAB_ERR_CAPACITY = -6
ARTAB_ERR_LAUNCH = -7

_DTYPE_CODE = {torch.bfloat16: ARTAB_BF16, torch.float16: ARTAB_F16, torch.float32: ARTAB_F32}


class ArtabView(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("stride_b", ctypes.c_int64),
        ("stride_h", ctypes.c_int64),
        ("stride_n", ctypes.c_int64),
    ]


_VP = ctypes.POINTER(ArtabView)
_i, _f, _p, _sz, _i64 = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int64


class ArtabAttentionPartials(ctypes.Structure):
    """``artab_attention_partials`` of include/artab_attention.h."""

    _fields_ = [("part_o", _p), ("part_lse", _p), ("n_slots", _i), ("B", _i), ("H", _i), ("Lq", _i), ("Dh", _i),
                ("order_state", _p), ("order_timeout_us", ctypes.c_uint64), ("order_flags", _i)]


class ArtabSampleEmbedArgs(ctypes.Structure):
    """``artab_sample_embed_args`` of include/artab_attention.h, field for field."""

    _fields_ = [
        ("x_last", _p), ("ld_row", _i64),
        ("norm_gamma", _p), ("norm_beta", _p), ("eps", _f),
        ("w_h1", _p), ("b_h1", _p), ("w_h2", _p), ("b_h2", _p),
        ("mean_bias", _p), ("std_bias", _p), ("weight_bias", _p),
        ("K", _i), ("std_min", _f), ("std_max", _f),
        ("rand_u", _p), ("rand_n", _p), ("x_mean", _p),
        ("w_x", _p), ("b_x", _p), ("w_y", _p), ("b_y", _p),
        ("markers", _p), ("ar_tokens", _p), ("bs", _i),
        ("step", _p), ("Nt", _i),
        ("preds", _p), ("emb_next", _p),
        ("B", _i), ("D", _i), ("F", _i),
        ("advance", _p), ("n_advance", _i), ("ticket", _p),
    ]


# name -> (restype, argtypes); every symbol declared in include/artab_attention.h
SIGNATURES = {
    "artab_version": (_i, []),
    "artab_status_string": (ctypes.c_char_p, [_i]),
    "artab_last_error": (ctypes.c_char_p, []),
    "artab_tuning_set": (_i, [ctypes.c_char_p, _i, _i]),
    "artab_tuning_get": (_i, [ctypes.c_char_p, ctypes.POINTER(_i)]),
    "artab_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i]),
    "artab_context_attention": (_i, [_VP, _VP, _VP, _VP, _p, _i, _i, _i, _i, _i, _f, _i, _p, _sz, _i, _p]),
    "artab_decode_attention": (
        _i,
        [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _i, _i, _i, _i, _i, _p, _i, _i, _f, _i, _p, _sz, _i, _p],
    ),
    "artab_decode_attention_static": (
        _i,
        [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _i, _i, _i, _i, _i, _p, _i, _i, _f, _i, _i, _p],
    ),
    "artab_decode_attention_overlapped": (
        _i,
        [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _i, _i, _i, _i, _i, _p, _i, _i, _f, _i, _p, _sz, _i, _p, _p],
    ),
    "artab_decode_attention_partials": (
        _i,
        [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _i, _i, _i, _i, _i, _p, _i, _i, _f, _i, _p, _sz, _i, _p, _p,
         ctypes.POINTER(ArtabAttentionPartials)],
    ),
    "artab_decode_attention_partials_ordered": (
        _i,
        [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _i, _i, _i, _i, _i, _p, _i, _i, _f, _i, _p, _sz, _i, _p, _p,
         ctypes.POINTER(ArtabAttentionPartials), _p, ctypes.c_uint64, _i],
    ),
    "artab_order_signal": (_i, [_p, _i, _p]),
    "artab_order_wait": (_i, [_p, _i, ctypes.c_uint64, _p]),
    "artab_teacher_forcing_attention": (_i, [_VP, _VP, _VP, _VP, _VP, _VP, _p, _i, _i, _i, _i, _i, _f, _i, _i, _p]),
    "artab_row_mask_attention": (_i, [_VP, _VP, _VP, _VP, _p, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _p]),
    "artab_row_mask_attention_backward": (
        _i, [_VP, _VP, _VP, _VP, _VP, _p, _p, _VP, _VP, _VP, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _p]),
    "artab_prefill_attention": (_i, [_VP, _VP, _VP, _VP, _VP, _VP, _i, _i, _i, _i, _i, _f, _i, _i, _p]),
    "artab_buffer_attention": (_i, [_VP, _VP, _VP, _p, _i64, _i64, _i64, _VP, _p, _i, _i, _i, _i, _i, _f, _i, _p]),
    "artab_merge_attention_outputs": (_i, [_VP, _p, _VP, _p, _VP, _i, _i, _i, _i, _i, _p]),
    "artab_add_layernorm": (_i, [_p, _i64, _p, _i64, _p, _p, _p, _p, _i64, _i, _f, _i, _p]),
    "artab_bias_gelu": (_i, [_p, _i64, _p, _p, _i64, _i, _i, _p]),
    "artab_pack_linear_weight": (_i, [_p, _p, _i, _i, _i, _p]),
    "artab_layer_pre": (_i, [_p, _i64, _p, _p, _p, _f, _p, _p, _p, _i64, _i, _i, _p]),
    "artab_layer_post_pre": (
        _i,
        [_p, _i64, _p, _i64, _p, _p, _p, _f, _p, _p, _p, _p, _p, _p, _f, _p, _p, _p, _f, _p, _p, _p, _i64, _i, _i, _i, _p],
    ),
    "artab_merge_attention_partials": (_i, [ctypes.POINTER(ArtabAttentionPartials), _VP, _i, _p]),
    "artab_layer_post_from_partials": (
        _i, [ctypes.POINTER(ArtabAttentionPartials), _p, _i64, _p, _p, _p, _f, _p, _p, _p, _p, _p, _p, _f, _p, _i64, _i, _i, _i, _p]),
    "artab_layer_post_pre_from_partials": (
        _i,
        [ctypes.POINTER(ArtabAttentionPartials), _p, _i64, _p, _p, _p, _f, _p, _p, _p, _p, _p, _p, _f, _p, _p, _p, _f, _p, _p, _p, _i64, _i, _i, _i, _p],
    ),
    "artab_decode_sample_embed": (_i, [ctypes.POINTER(ArtabSampleEmbedArgs), _i, _p]),
    "artab_decode_step_boundary": (
        _i,
        [ctypes.POINTER(ArtabAttentionPartials), _p, _i64, _p, _i64, _p, _p, _p, _f, _p, _p, _p, _p, _p, _p, _f,
         ctypes.POINTER(ArtabSampleEmbedArgs), _p, _p, _p, _f, _p, _p, _p, _i, _i, _p],
    ),
    "artab_layer_post": (_i, [_p, _i64, _p, _i64, _p, _p, _p, _f, _p, _p, _p, _p, _p, _p, _f, _p, _i64, _i, _i, _i, _p]),
}

# every symbol declared in include/artab_bench.h (exported by libartab_bench.so only)
BENCH_SIGNATURES = {
    "artab_profile_begin": (_i, [_i]),
    "artab_profile_end": (_i, [ctypes.POINTER(_f), ctypes.POINTER(_i), _i]),
    "artab_stamps_begin": (_i, [_i]),
    "artab_stamps_end": (_i, [ctypes.POINTER(_f), _i]),
    "artab_bench_instruction_mix": (_i, [_i, _i, _i, _i, _sz, _p, _p, _p]),
}

TUNING_KEYS = ("ARTAB_BM", "ARTAB_SPLIT", "ARTAB_SMALL", "ARTAB_STREAM", "ARTAB_STREAM_PER_CU", "ARTAB_STREAM_PRIO",
               "ARTAB_STREAM_SHORT", "ARTAB_STREAM_CALM", "ARTAB_DENSE_BELOW", "ARTAB_CTX_YIELD", "ARTAB_ORDER_GATE_LAUNCH", "ARTAB_BN", "ARTAB_LEAN",
               "ARTAB_LEAN_OCC", "ARTAB_NW", "ARTAB_TILE_ROWS", "ARTAB_LAYER_FETCHERS")

_lib: Optional[ctypes.CDLL] = None
_product_lib: Optional[ctypes.CDLL] = None
_bench_lib: Optional[ctypes.CDLL] = None


def library_built() -> bool:
    return os.path.exists(LIB_PATH)


def _open(path: str, signatures) -> ctypes.CDLL:
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: the HIP extension has not been built. "
            "Build it with `python -m ar_nanotabpfn_amd.build_ext` (needs hipcc, targets gfx950). "
            "There is no CPU fallback for the attention path."
        )
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in signatures.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.artab_version() != ABI_VERSION:
        raise RuntimeError(f"{path}: ABI version {lib.artab_version()} != {ABI_VERSION}; rebuild the extension")
    return lib


def load() -> ctypes.CDLL:
    """Load the shared library once; raise loudly when it is missing."""
    global _lib, _product_lib
    if _lib is not None:
        return _lib
    _product_lib = _open(LIB_PATH, SIGNATURES)
    _lib = _product_lib
    return _lib


class benchmark_library:
    """``with benchmark_library() as lib:`` — every call of this package goes through
    ``libartab_bench.so`` inside the block (same kernels, plus the aids of include/artab_bench.h
    on ``lib``), and through the product library again afterwards.  Overrides set with
    ``tuning`` belong to the library they were set on."""

    def __enter__(self) -> ctypes.CDLL:
        global _lib, _bench_lib
        load()
        if _bench_lib is None:
            _bench_lib = _open(BENCH_LIB_PATH, {**SIGNATURES, **BENCH_SIGNATURES})
        _lib = _bench_lib
        return _bench_lib

    def __exit__(self, *exc):
        global _lib
        _lib = _product_lib
        return False


class tuning:
    """``with tuning(ARTAB_SMALL=0, ARTAB_TILE_ROWS=16):`` sets route overrides of the loaded
    library (``artab_tuning_set``) and restores the previous state on exit; ``None`` removes an
    override.  ``tuning.set(...)`` / ``tuning.get(name)`` for callers that manage the lifetime
    themselves (pytest fixtures)."""

    def __init__(self, **overrides):
        self.overrides = overrides
        self.saved = {}

    @staticmethod
    def get(name: str) -> Optional[int]:
        v = _i(0)
        rc = load().artab_tuning_get(name.encode(), ctypes.byref(v))
        if rc < 0:
            check(rc)
        return int(v.value) if rc == 1 else None

    @staticmethod
    def set(**overrides) -> None:
        lib = load()
        for name, value in overrides.items():
            if value is None:
                check(lib.artab_tuning_set(name.encode(), 0, 0))
            else:
                check(lib.artab_tuning_set(name.encode(), int(value), 1))

    def __enter__(self):
        self.saved = {k: tuning.get(k) for k in self.overrides}
        tuning.set(**self.overrides)
        return self

    def __exit__(self, *exc):
        tuning.set(**self.saved)
        return False


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}; expected bfloat16, float16 or float32") from None


def require_device(*tensors: Optional[torch.Tensor]) -> torch.device:
    """All given tensors must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "ar_nanotabpfn_amd attention runs on a HIP device only (got a tensor on "
                f"{t.device}); there is no CPU implementation in this package."
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError(f"tensors on different devices: {dev} and {t.device}")
    if dev is None:
        raise ValueError("no tensor given")
    return dev


def view4(t: Optional[torch.Tensor], shared_batch: bool = False) -> Optional[ArtabView]:
    """Describe a ``[B,H,N,Dh]`` tensor (or ``[H,N,Dh]`` with ``shared_batch``) for the C ABI."""
    if t is None:
        return None
    if shared_batch:
        if t.dim() != 3:
            raise ValueError(f"expected a [H,N,Dh] tensor, got {tuple(t.shape)}")
        if t.shape[-1] > 1 and t.stride(-1) != 1:
            raise ValueError("head_dim axis must be contiguous")
        return ArtabView(t.data_ptr(), 0, t.stride(0), t.stride(1))
    if t.dim() != 4:
        raise ValueError(f"expected a [B,H,N,Dh] tensor, got {tuple(t.shape)}")
    if t.shape[-1] > 1 and t.stride(-1) != 1:
        raise ValueError("head_dim axis must be contiguous")
    return ArtabView(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def ref(v: Optional[ArtabView]):
    return ctypes.byref(v) if v is not None else None


def current_stream(device: torch.device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def check(status: int) -> None:
    """Map a negative status to the exception the reference raises for that condition:
    ``ValueError`` for shape/contract violations, ``RuntimeError`` for device-side
    unavailability or launch failure."""
    if status == 0:
        return
    lib = load()
    msg = lib.artab_last_error().decode() or lib.artab_status_string(status).decode()
    if status in (ARTAB_ERR_BAD_SHAPE, ARTAB_ERR_CAPACITY, ARTAB_ERR_BAD_STRIDE, ARTAB_ERR_NULL_POINTER):
        raise ValueError(msg)
    raise RuntimeError(msg)


_workspaces = {}
_workspace_tag = 0


class workspace_tag:
    """Calls made inside ``with workspace_tag(i):`` use scratch tensor ``i`` of their device.
    Launch sequences that run concurrently on different streams (each ordered in itself) must not
    share one: give each its own tag."""

    def __init__(self, tag: int):
        self.tag = int(tag)

    def __enter__(self):
        global _workspace_tag
        self.prev, _workspace_tag = _workspace_tag, self.tag
        return self

    def __exit__(self, *exc):
        global _workspace_tag
        _workspace_tag = self.prev
        return False


def workspace(device: torch.device, nbytes: int) -> Optional[torch.Tensor]:
    """A float32 scratch tensor of at least ``nbytes`` on ``device`` (grown on demand,
    reused between calls: consecutive launches on one stream are ordered)."""
    if nbytes <= 0:
        return None
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device(), _workspace_tag)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() * 4 < nbytes:
        # the outgrown tensor is dropped here; whoever recorded launches that point at it (a HIP
        # graph) keeps it alive through ``held_workspace``
        ws = torch.empty((nbytes + 3) // 4, device=device, dtype=torch.float32)
        _workspaces[key] = ws
    return ws


def held_workspace(device: torch.device, tag: Optional[int] = None) -> Optional[torch.Tensor]:
    """The scratch tensor that calls on ``device`` under ``tag`` (default: the current tag) use at
    the moment.  A caller that records such calls into a HIP graph keeps the returned tensor for as
    long as the graph lives: the module itself lets go of a scratch tensor when a larger one is
    needed."""
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device(),
           _workspace_tag if tag is None else int(tag))
    return _workspaces.get(key)
