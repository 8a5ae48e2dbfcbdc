"""ctypes binding of libpiper_amd.so (declared in include/piper_amd.h).

The library is loaded lazily on first use and never silently replaced: if it has not been
built, or a call returns a non-zero status, a RuntimeError is raised.  This mirrors the
reference, where every failure inside a task is a Python exception that propagates to the
driver (e.g. the assertions in src/runtime.py:313-328).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "libpiper_amd.so"

PK_F32 = 0
PK_BF16 = 1

_c_i64 = C.c_int64
_c_int = C.c_int
_c_f32 = C.c_float
_p = C.c_void_p

# name -> (restype, argtypes); must list every symbol declared in include/piper_amd.h
SIGNATURES = {
    "pk_version": (_c_int, []),
    "pk_status_string": (C.c_char_p, [_c_int]),
    "pk_init": (_c_int, []),
    "pk_sched_slot_index": (_c_int, [_c_int, C.c_uint64, C.c_uint64, C.c_uint64]),
    "pk_gate_workspace_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "pk_gate_logits": (_c_int, [_p, _c_int, _p, _p, _p, _c_i64, _c_i64, _c_i64, _p, _c_i64, _p]),
    "pk_route_topk": (_c_int, [_p, _c_i64, _c_i64, _c_i64, _c_int, _c_f32, _p, _p, _p]),
    "pk_route_topk_bwd": (_c_int, [_p, _p, _p, _c_i64, _c_i64, _c_i64, _c_int, _c_f32, _p, _p]),
    "pk_gate_bwd_workspace_bytes": (_c_i64, [_c_i64, _c_i64, _c_i64]),
    "pk_gate_logits_bwd": (_c_int, [_p, _p, _c_int, _p, _p, _p, _p, _c_int, _c_i64, _c_i64, _c_i64, _p, _c_i64, _p]),
    "pk_sort_workspace_bytes": (_c_i64, [_c_i64, _c_i64]),
    "pk_sort_by_expert": (_c_int, [_p, _c_i64, _c_i64, _p, _p, _p, _p, _p, _p, _c_i64, _p]),
    "pk_sort_by_expert_static": (_c_int, [_p, _c_i64, _c_i64, _p, _p, _p, _p, _p, _p]),
    "pk_counts_to_starts": (_c_int, [_p, _c_int, _c_i64, _p, _p]),
    "pk_permute_fwd": (_c_int, [_p, _c_int, _p, _p, _c_i64, _c_i64, _c_i64, _p]),
    "pk_permute_bwd": (_c_int, [_p, _c_int, _p, _p, _p, _c_i64, _c_i64, _c_i64, _p]),
    "pk_combine_fwd": (_c_int, [_p, _c_int, _p, _p, _p, _p, _c_i64, _c_i64, _c_i64, _p]),
    "pk_rmsnorm_fwd": (_c_int, [_p, _c_int, _p, _c_f32, _p, _p, _c_i64, _c_i64, _p]),
    "pk_rmsnorm_bwd_workspace_bytes": (_c_i64, [_c_i64, _c_i64]),
    "pk_rmsnorm_bwd": (_c_int, [_p, _p, _c_int, _p, _p, _p, _p, _p, _c_int, _c_i64, _c_i64, _p, _c_i64, _p]),
    "pk_combine_bwd": (_c_int, [_p, _p, _c_int, _p, _p, _p, _p, _c_i64, _c_i64, _c_i64, _p]),
    "pk_zero_rows_from": (_c_int, [_p, _c_int, _p, _c_i64, _c_i64, _p]),
    "pk_grouped_swiglu_fwd": (_c_int, [_p, _p, _c_i64, _p, _p, _p, _p, _p, _p, _p, _p,
                                       _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_grouped_swiglu_dgrad": (_c_int, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p,
                                         _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_grouped_swiglu_dgrad_dh": (_c_int, [_p, _p, _p, _p, _p, _p, _p, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_grouped_swiglu_dgrad_dx": (_c_int, [_p, _p, _p, _p, _p, _p, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_grouped_swiglu_wgrad": (_c_int, [_p, _p, _p, _p, _p, _p, _c_i64, _p, _p, _p, _p, _p, _c_int,
                                         _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_grouped_swiglu_wgrad_scaled": (_c_int, [_p, _p, _p, _p, _p, _p, _c_i64, _p, _p, _p, _p, _p, _c_int,
                                                _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes": (_c_i64, [_c_i64, _c_i64]),
    "pk_grouped_swiglu_dgrad_dh_scaled": (_c_int, [_p, _p, _c_i64, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _c_i64,
                                                   _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_grouped_swiglu_transposed_ld": (_c_i64, [_c_i64, _c_i64, _c_i64, _c_i64, _c_int]),
    # d_out row_map div scores w2 g u starts d_g d_u d_gT d_uT hsT ldt d_scores ws ws_bytes A H I E dtype stream
    "pk_grouped_swiglu_dgrad_dh_scaled_t": (_c_int, [_p, _p, _c_i64, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _c_i64, _p,
                                                     _p, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_grouped_swiglu_dx_from_transposed_pays": (_c_int, [_c_i64, _c_i64, _c_i64, _c_i64, _c_int]),
    "pk_grouped_swiglu_dgrad_dx_t": (_c_int, [_p, _p, _c_i64, _p, _p, _p, _p, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    # d_out hsT d_gT d_uT ldt x row_map div starts order d_w1 d_w2 d_w3 accumulate A H I E dtype stream
    "pk_grouped_swiglu_wgrad_scaled_t": (_c_int, [_p, _p, _p, _p, _c_i64, _p, _p, _c_i64, _p, _p, _p, _p, _p, _c_int,
                                                  _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _p]),
    "pk_bucket_plan": (_c_i64, [_p, _c_i64, _c_i64, _c_i64, _p]),
    "pk_bucket_pack": (_c_int, [_p, _p, _p, _c_i64, _c_int, _p, _c_int, _c_int, _p]),
    "pk_bucket_unpack": (_c_int, [_p, _c_int, _p, _p, _p, _c_i64, _c_int, _p]),
    "pk_bucket_zero": (_c_int, [_p, _c_i64, _p]),
    "pk_adamw_fused": (_c_int, [_p, _p, _p, _p, _p, _c_int, _c_i64, _c_f32, _c_f32, _c_f32, _c_f32,
                                _c_f32, _c_i64, _c_f32, _c_int, _p]),
    "pk_adamw_fused_packed": (_c_int, [_p, _p, _p, _p, _p, _p, _p, _c_i64, _c_int, _p, _c_int, _c_f32, _c_f32, _c_f32,
                                       _c_f32, _c_f32, _c_i64, _c_f32, _c_int, _p]),
    "pk_timing_enable": (_c_int, [_c_int]),
    "pk_timing_collect": (_c_i64, [_p, _p, _c_i64]),
    "pk_timing_select": (_c_int, [_c_int]),
    "pk_timing_kernel_name": (C.c_char_p, [_c_int]),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m piper_amd.build` "
                "(there is no fallback implementation)"
            )
        lib = C.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError here means header and library disagree
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def is_built() -> bool:
    return LIB_PATH.exists()


def status_string(status: int) -> str:
    return load().pk_status_string(int(status)).decode()


_ready_devices: set = set()


def init_device() -> None:
    """pk_init() once per device: the library's device arrays are resolved before any launch, so
    that the first launch of an entry point may already sit inside a HIP graph capture."""
    dev = torch.cuda.current_device()
    if dev in _ready_devices:
        return
    rc = load().pk_init()
    if rc != 0:
        raise RuntimeError(f"pk_init failed with status {rc}: {status_string(rc)}")
    _ready_devices.add(dev)


def call(name: str, *args):
    """Call an int-returning entry point and raise RuntimeError on a non-zero status."""
    rc = getattr(load(), name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed with status {rc}: {status_string(rc)}")
    return rc


def timing_enable(on: bool) -> None:
    """Switch per-kernel HIP-event timing inside the library on or off."""
    load().pk_timing_enable(int(bool(on)))


def timing_select(name: str | None) -> None:
    """Time only the kernel with this name (as timing_collect reports it); None times all again."""
    lib = load()
    kid = -1
    if name is not None:
        i = 0
        while True:
            n = lib.pk_timing_kernel_name(i).decode()
            if n == "unknown":
                raise ValueError(f"no kernel named {name!r}")
            if n == name:
                kid = i
                break
            i += 1
    lib.pk_timing_select(kid)


def timing_collect(max_records: int = 1 << 16) -> list[tuple[str, float]]:
    """Wait for and return the (kernel name, milliseconds) records since the last collect."""
    lib = load()
    ids = (C.c_int32 * max_records)()
    ms = (C.c_float * max_records)()
    n = min(int(lib.pk_timing_collect(ids, ms, max_records)), max_records)
    return [(lib.pk_timing_kernel_name(ids[i]).decode(), float(ms[i])) for i in range(n)]


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return PK_F32
    if dtype == torch.bfloat16:
        return PK_BF16
    raise TypeError(f"piper_amd kernels support float32 and bfloat16, got {dtype}")


def ptr(t: torch.Tensor | None):
    """Device pointer of a contiguous tensor (None -> NULL)."""
    if t is None:
        return None
    if not t.is_contiguous():
        raise ValueError("piper_amd kernels need contiguous tensors")
    return t.data_ptr()


def current_stream(device: torch.device | None = None):
    """The hipStream_t of torch's current stream, so kernels respect `torch.cuda.stream(...)`
    exactly like the ATen ops they replace (src/executors.py:231-232)."""
    init_device()
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            "piper_amd kernels run on the GPU only; got a tensor on "
            f"{t.device} (there is no CPU fallback)"
        )
