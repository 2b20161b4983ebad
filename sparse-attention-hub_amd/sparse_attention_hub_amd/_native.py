"""ctypes binding of libsah_mi355.so (declared in include/sah.h).

The library is the only compute back end of this package: every masker and the
masked attention call into it, and a missing library is an error, not a reason
to fall back to torch. PyTorch is used for device memory and the current
stream only.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path
from typing import Optional

import torch

_PKG_ROOT = Path(__file__).resolve().parent.parent  # sparse-attention-hub_amd/
_DEFAULT_LIB = _PKG_ROOT / "lib" / "libsah_mi355.so"

# SAH_VERSION of the include/sah.h the structures below were written against
ABI_VERSION = 4

SAH_F32, SAH_BF16, SAH_F16 = 0, 1, 2
SAH_ACT = {"relu": 0, "silu": 1, "gelu": 2, "tanh": 3}
SAH_MAX_MLP_LAYERS = 4

_DTYPE_CODE = {torch.float32: SAH_F32, torch.bfloat16: SAH_BF16, torch.float16: SAH_F16}

EXPECTED_SYMBOLS = (
    "sah_version",
    "sah_last_error",
    "sah_timing_enable",
    "sah_timing_collect",
    "sah_sink_local_indices",
    "sah_rows_from_dense",
    "sah_rows_to_dense",
    "sah_hash_signatures",
    "sah_hash_signatures_pair",
    "sah_hamming_topk",
    "sah_hamming_scores",
    "sah_hash_decode_topk",
    "sah_hash_decode_attention",
    "sah_hash_compact_codes",
    "sah_qk_scores",
    "sah_select_topk",
    "sah_pq_keys_absmax",
    "sah_pq_kmeans_assign",
    "sah_pq_kmeans_update",
    "sah_pq_adc_scores",
    "sah_pq_adc_lut_bytes",
    "sah_adaptive_budget",
    "sah_adaptive_sample",
    "sah_sparse_attention_work_floats",
    "sah_sparse_attention",
    "sah_sparse_attention_static",
    "sah_attention_weights",
    "sah_run_chain",
    "sah_amask_classify",
    "sah_select_topk_attention",
)


class NativeLibraryError(RuntimeError):
    """libsah_mi355.so is missing, stale or returned an error."""


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}; expected float32, bfloat16 or float16") from None


class Rows(C.Structure):
    _fields_ = [
        ("cols", C.c_void_p),
        ("cnt", C.c_void_p),
        ("w", C.c_void_p),
        ("bitmap", C.c_void_p),
        ("n_rows", C.c_int32),
        ("cap", C.c_int32),
        ("n_keys", C.c_int32),
        ("n_words", C.c_int32),
    ]


class SinkLocalArgs(C.Structure):
    _fields_ = [
        ("rows", Rows),
        ("lq", C.c_int32),
        ("sink", C.c_int32),
        ("window", C.c_int32),
        ("fresh", C.c_int32),
        ("clear_future", C.c_int32),
        ("stream", C.c_void_p),
    ]


class DenseRowsArgs(C.Structure):
    _fields_ = [("rows", Rows), ("dense", C.c_void_p), ("dtype", C.c_int32), ("stream", C.c_void_p)]


class HashSigArgs(C.Structure):
    _fields_ = [
        ("x", C.c_void_p),
        ("xs_b", C.c_int64), ("xs_h", C.c_int64), ("xs_l", C.c_int64),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hq", C.c_int32), ("group", C.c_int32), ("L", C.c_int32), ("D", C.c_int32),
        ("n_layers", C.c_int32),
        ("W", C.c_void_p * SAH_MAX_MLP_LAYERS),
        ("bias", C.c_void_p * SAH_MAX_MLP_LAYERS),
        ("Wt", C.c_void_p * SAH_MAX_MLP_LAYERS),
        ("d_out", C.c_int32 * SAH_MAX_MLP_LAYERS),
        ("act", C.c_int32),
        ("codes", C.c_void_p),
        ("code_pitch", C.c_int64),
        ("code_offset", C.c_int64),
        ("stream", C.c_void_p),
    ]


class HammingTopkArgs(C.Structure):
    _fields_ = [
        ("rows", Rows),
        ("kcodes", C.c_void_p),
        ("code_pitch", C.c_int64),
        ("qcodes", C.c_void_p),
        ("lq", C.c_int32),
        ("k", C.c_int32),
        ("stream", C.c_void_p),
    ]


class HammingScoresArgs(C.Structure):
    _fields_ = [
        ("kcodes", C.c_void_p),
        ("code_pitch", C.c_int64),
        ("qcodes", C.c_void_p),
        ("B", C.c_int32), ("Hq", C.c_int32), ("Lq", C.c_int32), ("n_keys", C.c_int32),
        ("amask", C.c_void_p), ("ms_b", C.c_int64), ("ms_h", C.c_int64), ("ms_l", C.c_int64),
        ("dtype", C.c_int32),
        ("keys_out", C.c_void_p),
        ("key_pitch", C.c_int64),
        ("stream", C.c_void_p),
    ]


class QkScoresArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("qs_b", C.c_int64), ("qs_h", C.c_int64), ("qs_l", C.c_int64),
        ("k", C.c_void_p), ("ks_b", C.c_int64), ("ks_h", C.c_int64), ("ks_l", C.c_int64),
        ("amask", C.c_void_p), ("ms_b", C.c_int64), ("ms_h", C.c_int64), ("ms_l", C.c_int64),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("Lq", C.c_int32), ("Lk", C.c_int32), ("D", C.c_int32),
        ("keys_out", C.c_void_p),
        ("key_pitch", C.c_int64),
        ("stream", C.c_void_p),
        ("resid_out", C.c_void_p),
    ]


class SelectTopkArgs(C.Structure):
    _fields_ = [
        ("rows", Rows),
        ("keys", C.c_void_p),
        ("key_pitch", C.c_int64),
        ("key_bits", C.c_int32),
        ("n_cand", C.c_int32),
        ("col_offset", C.c_int32),
        ("k", C.c_int32),
        ("excluded_key", C.c_uint32),
        ("fresh", C.c_int32),
        ("fresh_sink", C.c_int32),
        ("fresh_window", C.c_int32),
        ("stream", C.c_void_p),
        ("skip_bitmap", C.c_int32),
    ]


class PqAssignArgs(C.Structure):
    _fields_ = [
        ("k", C.c_void_p), ("ks_b", C.c_int64), ("ks_h", C.c_int64), ("ks_l", C.c_int64),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hkv", C.c_int32), ("n_sub", C.c_int32), ("d_sub", C.c_int32), ("n_cent", C.c_int32),
        ("key_offset", C.c_int32), ("n_keys", C.c_int32),
        ("centres", C.c_void_p),
        ("codes", C.c_void_p), ("code_pitch", C.c_int64), ("code_offset", C.c_int64),
        ("sums", C.c_void_p), ("counts", C.c_void_p),
        ("round_dist", C.c_int32),
        ("skip_flag", C.c_void_p),
        ("stream", C.c_void_p),
        ("absmax_bits", C.c_void_p),
    ]


class PqUpdateArgs(C.Structure):
    _fields_ = [
        ("k", C.c_void_p), ("ks_b", C.c_int64), ("ks_h", C.c_int64), ("ks_l", C.c_int64),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hkv", C.c_int32), ("n_sub", C.c_int32), ("d_sub", C.c_int32), ("n_cent", C.c_int32),
        ("key_offset", C.c_int32),
        ("centres", C.c_void_p),
        ("sums", C.c_void_p), ("counts", C.c_void_p),
        ("reseed_idx", C.c_void_p),
        ("shift2", C.c_void_p),
        ("tol", C.c_float),
        ("state", C.c_void_p),
        ("stream", C.c_void_p),
        ("absmax_bits", C.c_void_p),
    ]


class PqAbsmaxArgs(C.Structure):
    _fields_ = [
        ("k", C.c_void_p), ("ks_b", C.c_int64), ("ks_h", C.c_int64), ("ks_l", C.c_int64),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hkv", C.c_int32), ("D", C.c_int32),
        ("key_offset", C.c_int32), ("n_keys", C.c_int32),
        ("absmax_bits", C.c_void_p),
        ("stream", C.c_void_p),
    ]


class PqAdcArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("qs_b", C.c_int64), ("qs_h", C.c_int64), ("qs_l", C.c_int64),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("Lq", C.c_int32),
        ("n_sub", C.c_int32), ("d_sub", C.c_int32), ("n_cent", C.c_int32),
        ("centres", C.c_void_p),
        ("codes", C.c_void_p), ("code_pitch", C.c_int64),
        ("n_cand", C.c_int32),
        ("keys_out", C.c_void_p), ("key_pitch", C.c_int64),
        ("lut", C.c_void_p), ("lut_bytes", C.c_int64),
        ("stream", C.c_void_p),
        ("centres_narrow", C.c_void_p),
    ]


class AdaptiveBudgetArgs(C.Structure):
    _fields_ = [
        ("rows", Rows),
        ("keys", C.c_void_p), ("key_pitch", C.c_int64),
        ("amask", C.c_void_p), ("ms_b", C.c_int64), ("ms_h", C.c_int64), ("ms_l", C.c_int64),
        ("dtype", C.c_int32),
        ("Hq", C.c_int32), ("Lq", C.c_int32),
        ("scaling", C.c_float),
        ("start", C.c_int32), ("range", C.c_int32), ("n_base", C.c_int32),
        ("eps", C.c_float), ("delta_ppf", C.c_float),
        ("seed", C.c_uint64), ("offset", C.c_uint64),
        ("prev_empty", C.c_int32),
        ("budget", C.c_void_p),
        ("prob", C.c_void_p),
        ("stats", C.c_void_p),
        ("stream", C.c_void_p),
        ("max_in_rows", C.c_int32),
    ]


class AdaptiveSampleArgs(C.Structure):
    _fields_ = [
        ("rows", Rows),
        ("budget", C.c_void_p),
        ("prob", C.c_void_p),
        ("dtype", C.c_int32),
        ("start", C.c_int32), ("range", C.c_int32),
        ("seed", C.c_uint64), ("offset", C.c_uint64),
        ("w_fresh", C.c_int32),
        ("stream", C.c_void_p),
    ]


class AttentionArgs(C.Structure):
    _fields_ = [
        ("rows", Rows),
        ("q", C.c_void_p), ("qs_b", C.c_int64), ("qs_h", C.c_int64), ("qs_l", C.c_int64),
        ("k", C.c_void_p), ("ks_b", C.c_int64), ("ks_h", C.c_int64), ("ks_l", C.c_int64),
        ("v", C.c_void_p), ("vs_b", C.c_int64), ("vs_h", C.c_int64), ("vs_l", C.c_int64),
        ("amask", C.c_void_p), ("ms_b", C.c_int64), ("ms_h", C.c_int64), ("ms_l", C.c_int64),
        ("sinks", C.c_void_p),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("Lq", C.c_int32), ("Lk", C.c_int32), ("D", C.c_int32),
        ("scaling", C.c_float),
        ("unit_inv_w", C.c_float),
        ("dense", C.c_int32),
        ("closed_form", C.c_int32),
        ("closed_sink", C.c_int32),
        ("closed_window", C.c_int32),
        ("max_cnt", C.c_int32),
        ("out", C.c_void_p),
        ("work", C.c_void_p), ("work_floats", C.c_int64),
        ("logits_out", C.c_void_p),
        ("stats_out", C.c_void_p),
        ("stream", C.c_void_p),
        ("dropout_p", C.c_float),
        ("dropout_seed", C.c_uint64),
        ("dropout_offset", C.c_uint64),
        ("dropout_numerator_only", C.c_int32),
        ("score_keys", C.c_void_p),
        ("score_resid", C.c_void_p),
        ("score_pitch", C.c_int64),
    ]


class HashDecodeArgs(C.Structure):
    _fields_ = [
        ("rows", Rows),
        ("sink", C.c_int32), ("window", C.c_int32),
        ("query_sig", C.c_void_p),
        ("key_sig", C.c_void_p),
        ("kcodes", C.c_void_p),
        ("code_pitch", C.c_int64),
        ("k", C.c_int32),
        ("skip_bitmap", C.c_int32),
        ("pos_codes", C.c_void_p),
        ("pos_pitch", C.c_int64),
        ("exc", C.c_void_p),
        ("exc_cnt", C.c_void_p),
        ("exc_cap", C.c_int32),
        ("full_plane", C.c_uint32),
        ("stream", C.c_void_p),
    ]


class HashCompactArgs(C.Structure):
    _fields_ = [
        ("codes", C.c_void_p),
        ("code_pitch", C.c_int64),
        ("n_rows", C.c_int32),
        ("from_", C.c_int32), ("to", C.c_int32),
        ("pos_codes", C.c_void_p),
        ("pos_pitch", C.c_int64),
        ("exc", C.c_void_p),
        ("exc_cap", C.c_int32),
        ("exc_cnt", C.c_void_p),
        ("full_plane", C.c_uint32),
        ("stream", C.c_void_p),
    ]


class ChainArgs(C.Structure):
    _fields_ = [
        ("sink_local", C.c_void_p),
        ("sig_a", C.c_void_p),
        ("sig_b", C.c_void_p),
        ("hamming", C.c_void_p),
        ("hash_decode", C.c_void_p),
        ("qk", C.c_void_p),
        ("pq_assign", C.c_void_p),
        ("pq_adc", C.c_void_p),
        ("select", C.c_void_p),
        ("attention", C.c_void_p),
        ("compact", C.c_void_p),
        ("tickets", C.c_void_p),
    ]


class AmaskClassifyArgs(C.Structure):
    _fields_ = [
        ("amask", C.c_void_p), ("ms_b", C.c_int64), ("ms_h", C.c_int64), ("ms_l", C.c_int64),
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hm", C.c_int32), ("Lq", C.c_int32), ("Lk", C.c_int32),
        ("flags", C.c_void_p),
        ("stream", C.c_void_p),
    ]


AMASK_NONZERO, AMASK_GENERAL = 1, 2


class AttentionWeightsArgs(C.Structure):
    _fields_ = [
        ("rows", Rows),
        ("logits", C.c_void_p),
        ("stats", C.c_void_p),
        ("unit_inv_w", C.c_float),
        ("dense", C.c_int32),
        ("dtype", C.c_int32),
        ("weights", C.c_void_p),
        ("stream", C.c_void_p),
        ("dropout_p", C.c_float),
        ("dropout_seed", C.c_uint64),
        ("dropout_offset", C.c_uint64),
    ]


_lib: Optional[C.CDLL] = None


def library_path() -> Path:
    override = os.environ.get("SAH_LIBRARY_PATH")
    return Path(override) if override else _DEFAULT_LIB


def lib() -> C.CDLL:
    """Load (once) and return the shared library; raise if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not path.exists():
        raise NativeLibraryError(
            f"{path} not found: build it with `python sparse-attention-hub_amd/build.py` "
            "(hipcc --offload-arch=gfx950). There is no fallback implementation."
        )
    try:
        handle = C.CDLL(str(path))
    except OSError as e:
        raise NativeLibraryError(f"cannot load {path}: {e}") from e
    missing = [s for s in EXPECTED_SYMBOLS if not hasattr(handle, s)]
    if missing:
        raise NativeLibraryError(f"{path} lacks symbols {missing}; rebuild it")
    handle.sah_version.restype = C.c_int
    found = int(handle.sah_version())
    if found != ABI_VERSION:
        raise NativeLibraryError(
            f"{path} is layout generation {found} of include/sah.h, this binding is generation {ABI_VERSION}: "
            "the argument structures would not match; rebuild the library from this tree")
    handle.sah_last_error.restype = C.c_char_p
    handle.sah_sparse_attention_work_floats.restype = C.c_int64
    handle.sah_sparse_attention_work_floats.argtypes = [C.c_int32, C.c_int32, C.c_int32]
    handle.sah_pq_adc_lut_bytes.restype = C.c_int64
    handle.sah_pq_adc_lut_bytes.argtypes = [C.c_int32] * 7
    for name in EXPECTED_SYMBOLS:
        if name in ("sah_version", "sah_last_error", "sah_sparse_attention_work_floats", "sah_pq_adc_lut_bytes",
                    "sah_timing_enable", "sah_timing_collect"):
            continue
        if name == "sah_hash_signatures_pair":
            getattr(handle, name).restype = C.c_int
            getattr(handle, name).argtypes = [C.c_void_p, C.c_void_p]
            continue
        if name in ("sah_select_topk_attention", "sah_hash_decode_attention"):
            getattr(handle, name).restype = C.c_int
            getattr(handle, name).argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
            continue
        fn = getattr(handle, name)
        fn.restype = C.c_int
        fn.argtypes = [C.c_void_p]
    _lib = handle
    return handle


def call(name: str, args: C.Structure) -> None:
    """Invoke an `int sah_*(const args*)` entry point and raise on a non-zero code."""
    handle = lib()
    rc = getattr(handle, name)(C.addressof(args))
    if rc != 0:
        msg = handle.sah_last_error().decode("utf-8", "replace")
        if rc in (-1, -3, -4, -5):
            raise ValueError(f"{name}: {msg} (code {rc})")
        raise NativeLibraryError(f"{name}: {msg} (code {rc})")


def call2(name: str, a: C.Structure, b: C.Structure) -> None:
    """Invoke an `int sah_*(const args*, const args*)` entry point and raise on a non-zero code."""
    handle = lib()
    rc = getattr(handle, name)(C.addressof(a), C.addressof(b))
    if rc != 0:
        msg = handle.sah_last_error().decode("utf-8", "replace")
        if rc in (-1, -3, -4, -5):
            raise ValueError(f"{name}: {msg} (code {rc})")
        raise NativeLibraryError(f"{name}: {msg} (code {rc})")


def timing_enable(on: bool) -> None:
    """Switch the library's per-kernel HIP-event timing on or off (benchmarks only)."""
    lib().sah_timing_enable(1 if on else 0)


def timing_collect(max_names: int = 64):
    """{kernel name: (launch count, total milliseconds)} since the last collect; waits for the events."""
    handle = lib()
    names = (C.c_char_p * max_names)()
    counts = (C.c_int * max_names)()
    total = (C.c_float * max_names)()
    handle.sah_timing_collect.restype = C.c_int
    n = handle.sah_timing_collect(names, counts, total, max_names)
    return {names[i].decode(): (int(counts[i]), float(total[i])) for i in range(n)}


def work_floats(n_rows: int, max_cnt: int, head_dim: int) -> int:
    return int(lib().sah_sparse_attention_work_floats(n_rows, max_cnt, head_dim))


def require_device(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise NativeLibraryError(
            f"{what} is on {t.device}: the MI355X kernels need GPU tensors and there is no CPU fallback"
        )


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device: torch.device) -> int:
    """The current stream of `device` as a hipStream_t (the kernels are launched on it)."""
    if device.type != "cuda":
        return 0
    if _RAW_STREAM is not None:  # the handle itself: no Stream object per call (5 us of a decode step's host time)
        index = device.index
        return int(_RAW_STREAM(torch.cuda.current_device() if index is None else index))
    return int(torch.cuda.current_stream(device).cuda_stream)


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()
