"""ctypes binding of liblfm2_hip.so (the C ABI declared in include/lfm2_hip.h).

There is no CPU fallback: if the library is missing or a call fails, an exception is raised.
Tensors are passed as raw device pointers; launches go to torch's current HIP stream so they are
ordered with torch's own work and are recorded by `torch.cuda.graph` captures.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "liblfm2_hip.so")

DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

# p = pointer, l = int64, i = int, f = float.  Order matches include/lfm2_hip.h.
_SIGNATURES = {
    "lfm2_embedding": "ppplllip",
    "lfm2_rms_norm": "ppppp" "llfip",
    "lfm2_embedding_rms_norm": "ppppppp" "lllfip",
    "lfm2_rms_norm_fp8": "pppppp" "llfip",
    "lfm2_swiglu": "ppllip",
    "lfm2_swiglu_fp8": "pppllip",
    "lfm2_quantize_rows": "pppllip",
    "lfm2_conv_update": "pppppp" "lllip",
    "lfm2_conv_update_fp8": "ppppppp" "lllip",
    "lfm2_prepare_qkv_store": "ppppppppppppp" "liiilflllii" "p",
    "lfm2_rms_norm_fp8_split": "pppp" "i" "pppp" "llfip",
    "lfm2_fp8_gemm_partials": "ppp" "llliip",
    "lfm2_fp8_gemm_qkv_store": "pppppppppppppppp" "liiillflllii" "p",
    "lfm2_bf16_gemm_partials": "ppp" "llliip",
    "lfm2_rms_norm_split": "ppp" "i" "pppp" "llfip",
    "lfm2_prepare_qkv": "ppppppppp" "liiilfip",
    "lfm2_conv_prefill": "ppppppp" "llllip",
    "lfm2_conv_prefill_fp8": "pppppppp" "llllip",
    "lfm2_fp8_gemm": "pppppp" "llliiip",
    "lfm2_bf16_gemm": "pppp" "llliip",
    "lfm2_fp8_gemm_rows": "ppppppp" "lllliip",
    "lfm2_fp8_gemm_swiglu": "ppppp" "llli" "p",
    "lfm2_bf16_gemm_swiglu": "ppp" "lll" "p",
    "lfm2_fp8_gemm_conv_update": "ppppppppp" "lllli" "p",
    "lfm2_bf16_gemm_conv_update": "ppppppp" "llll" "p",
    "lfm2_bf16_gemm_rows": "ppppp" "llllip",
    "lfm2_store_kv_fp8": "ppppppppp" "lliilllllllllip",
    "lfm2_append_kv": "ppppppp" "liilllip",
    "lfm2_store_kv_packed": "ppppppppp" "liillliip",
    "lfm2_decode_attention": "pppppppppp" "lipp" "liiillllfiippp",
    "lfm2_decode_schedule": "pppp" "lp",
    "lfm2_decode_begin": "pppppppp" "lp",
    "lfm2_prefill_attention": "ppppp" "lliiifip",
    "lfm2_build_token_map": "ppp" "llp",
    "lfm2_gather_inputs": "ppppppp" "lp",
    "lfm2_scatter_logits": "pppp" "llip",
    "lfm2_advance_positions": "pppp" "lp",
    "lfm2_sample": "pppppppp" "llfllip",
    "lfm2_sample_static": "pppppp" "llfllip",
    "lfm2_sample_filtered": "pppppppppp" "llfifllip",
    "lfm2_configure_rows": "p" "ll" "ppppppppppppp" "p",
    "lfm2_head_logprobs": "ppppp" "lliip",
    "lfm2_record_sample": "ppppppppppppppp" "llllp",
    "lfm2_sample_record": "pppppppppppppppppppp" "llllip",
    "lfm2_record_head": "pppppp" "illp",
    "lfm2_hbm_stream_read": "plpiip",
    "lfm2_mfma_fp8_peak": "ppiiip",
    "lfm2_timestamp": "pp",
}
_INT64_RESULT = {
    "lfm2_fp8_gemm_workspace": "lll",
    "lfm2_gemm_swiglu_fits": "llli",
    "lfm2_gemm_conv_fits": "llli",
    "lfm2_fp8_gemm_default_splits": "lll",
    "lfm2_bf16_gemm_default_splits": "lll",
    "lfm2_bf16_gemm_workspace": "lll",
    "lfm2_decode_attention_workspace": "liil",
    "lfm2_decode_schedule_size": "ll",
    "lfm2_timestamp_rate_khz": "",
}
_CTYPE = {"p": ctypes.c_void_p, "l": ctypes.c_int64, "i": ctypes.c_int, "f": ctypes.c_float}

_lib = None


def exported_symbols():
    """Every entry point include/lfm2_hip.h declares."""
    return sorted([*_SIGNATURES, *_INT64_RESULT, "lfm2_last_error", "lfm2_abi_version"])


def load():
    """Load the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY_PATH):
        raise RuntimeError(
            f"{LIBRARY_PATH} is missing: build it with `python -m climbing_gym_amd.build` (hipcc, gfx950). "
            "This package has no CPU or PyTorch fallback for its kernels.")
    lib = ctypes.CDLL(LIBRARY_PATH)
    for name, sig in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = [_CTYPE[c] for c in sig]
        fn.restype = ctypes.c_int
    for name, sig in _INT64_RESULT.items():
        fn = getattr(lib, name)
        fn.argtypes = [_CTYPE[c] for c in sig]
        fn.restype = ctypes.c_int64
    lib.lfm2_last_error.restype = ctypes.c_char_p
    lib.lfm2_abi_version.restype = ctypes.c_int
    _lib = lib
    return lib


def _arg(value):
    if value is None:
        return None
    if isinstance(value, torch.Tensor):
        return value.data_ptr()
    return value


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def stream_handle() -> int:
    """torch's current stream on the current device (the capture stream under `torch.cuda.graph`).  The raw accessors
    cost a fraction of a microsecond; `torch.cuda.current_stream()` builds a Stream object on every call, which at a
    hundred launches per prefill chunk is a visible share of the host time."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def call(name: str, *args):
    """Invoke an int-returning entry point on the current stream (appended as the last argument)."""
    lib = load()
    status = getattr(lib, name)(*[_arg(a) for a in args], stream_handle())
    if status != 0:
        message = lib.lfm2_last_error().decode()
        if status == -1:
            raise ValueError(f"{name}: {message}")
        raise RuntimeError(f"{name} failed ({status}): {message}")


def query(name: str, *args) -> int:
    return int(getattr(load(), name)(*args))


def require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("HIP kernels require tensors on the GPU")
