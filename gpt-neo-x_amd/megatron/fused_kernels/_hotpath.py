"""ctypes binding of libneox_hotpath.so (the C ABI declared in include/neox_hotpath.h).

The library is the only implementation: if it cannot be loaded an ImportError
is raised, there is no fallback of any kind.
"""
import ctypes
import os
import subprocess
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libneox_hotpath.so")
CSRC_DIR = os.path.normpath(os.path.join(_HERE, "..", "..", "csrc"))

F16, BF16, F32 = 0, 1, 2
_DTYPE = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}

ABI_VERSION = 1

_lock = threading.Lock()
_lib = None


def build(force=False, verbose=False):
    """Compile the HIP sources for gfx950 with hipcc (``make`` in csrc/)."""
    cmd = ["make", "-C", CSRC_DIR, "-j4"] + (["-B"] if force else [])
    out = None if verbose else subprocess.DEVNULL
    subprocess.run(cmd, check=True, stdout=out, stderr=None if verbose else subprocess.PIPE)
    return LIB_PATH


def _declare(lib):
    i64, vp, f32, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_int
    p64 = ctypes.POINTER(i64)
    u64, pu32 = ctypes.c_uint64, ctypes.POINTER(ctypes.c_uint32)
    sigs = {
        "nhp_abi_version": ([], ci),
        "nhp_status_string": ([ci], ctypes.c_char_p),
        "nhp_softmax_max_resident_row": ([], i64),
        "nhp_softmax_geometry": ([i64, ci, ctypes.POINTER(ci), ctypes.POINTER(ci), ctypes.POINTER(ci)], ci),
        "nhp_causal_softmax_fwd": ([vp, vp, f32, i64, i64, ci, vp], ci),
        "nhp_causal_softmax_bwd": ([vp, vp, vp, f32, i64, i64, ci, vp], ci),
        "nhp_causal_softmax_ex_fwd": ([vp, vp, f32, i64, i64, i64, vp, vp, vp, i64, ci, vp], ci),
        "nhp_causal_softmax_ex_bwd": ([vp, vp, vp, f32, i64, i64, i64, vp, i64, ci, vp], ci),
        "nhp_causal_softmax_dropout_fwd": ([vp, vp, vp, f32, i64, i64, i64, f32, u64, u64, ci, vp], ci),
        "nhp_causal_softmax_dropout_bwd": ([vp, vp, vp, f32, i64, i64, i64, f32, u64, u64, ci, vp], ci),
        "nhp_causal_softmax_blocks_fwd": ([vp, vp, f32, i64, i64, i64, i64, vp, vp, vp, i64, ci, vp], ci),
        "nhp_causal_softmax_blocks_bwd": ([vp, vp, vp, f32, i64, i64, i64, i64, vp, i64, ci, vp], ci),
        "nhp_causal_softmax_dropout_blocks_fwd": ([vp, vp, vp, f32, i64, i64, i64, i64, f32, u64, u64, ci, vp], ci),
        "nhp_causal_softmax_dropout_blocks_bwd": ([vp, vp, vp, f32, i64, i64, i64, i64, f32, u64, u64, ci, vp], ci),
        "nhp_masked_softmax_dropout_fwd": ([vp, vp, vp, vp, f32, i64, i64, i64, i64, i64, f32, u64, u64, ci, vp], ci),
        "nhp_masked_softmax_dropout_bwd": ([vp, vp, vp, f32, i64, i64, f32, u64, u64, ci, vp], ci),
        "nhp_masked_softmax_fwd": ([vp, vp, vp, f32, i64, i64, i64, i64, i64, ci, vp], ci),
        "nhp_masked_softmax_ex_fwd": ([vp, vp, vp, f32, i64, i64, i64, i64, i64, vp, vp, vp, ci, vp], ci),
        "nhp_masked_softmax_ex_dropout_fwd": ([vp, vp, vp, vp, f32, i64, i64, i64, i64, i64, vp, vp, vp, f32, u64, u64, ci, vp], ci),
        "nhp_causal_softmax_ex_dropout_fwd": ([vp, vp, vp, f32, i64, i64, i64, i64, vp, vp, vp, i64, f32, u64, u64, ci, vp], ci),
        "nhp_causal_softmax_ex_dropout_bwd": ([vp, vp, vp, f32, i64, i64, i64, i64, vp, i64, f32, u64, u64, ci, vp], ci),
        "nhp_masked_softmax_bwd": ([vp, vp, vp, f32, i64, i64, ci, vp], ci),
        "nhp_softmax_batch_per_block": ([i64, i64, i64, i64], ci),
        "nhp_rope_cached_fwd": ([vp, vp, vp, vp, i64, i64, i64, i64, i64, p64, p64, ci, ci, vp], ci),
        "nhp_rope_cached_bwd": ([vp, vp, vp, vp, i64, i64, i64, i64, i64, p64, p64, ci, ci, vp], ci),
        "nhp_rope_cached_qk_fwd": ([vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, p64, p64, p64, p64, ci, ci, vp], ci),
        "nhp_rope_cached_qk_bwd": ([vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, p64, p64, p64, p64, ci, ci, vp], ci),
        "nhp_rope_freqs_qk_fwd": ([vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, p64, p64, p64, p64, ci, vp], ci),
        "nhp_rope_freqs_qk_bwd": ([vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, p64, p64, p64, p64, ci, vp], ci),
        "nhp_rope_freqs_fwd": ([vp, vp, vp, i64, i64, i64, i64, i64, p64, p64, ci, vp], ci),
        "nhp_rope_freqs_bwd": ([vp, vp, vp, i64, i64, i64, i64, i64, p64, p64, ci, vp], ci),
        "nhp_bias_gelu_fwd": ([vp, vp, vp, i64, i64, ci, vp], ci),
        "nhp_bias_gelu_bwd": ([vp, vp, vp, vp, vp, vp, i64, i64, ci, vp], ci),
        "nhp_bias_gelu_bwd_workspace_bytes": ([i64, i64, ci], i64),
        "nhp_bias_add_residual": ([vp, vp, vp, vp, i64, i64, ci, vp], ci),
        "nhp_bias_add_residual_pair": ([vp, vp, vp, vp, vp, vp, i64, i64, ci, vp], ci),
        "nhp_bias_dropout_add": ([vp, vp, vp, vp, i64, i64, f32, u64, u64, ci, vp], ci),
        "nhp_dropout_bwd": ([vp, vp, i64, i64, f32, u64, u64, ci, vp], ci),
        "nhp_philox4x32_10": ([pu32, pu32, pu32], None),
        "nhp_gated_act_fwd": ([vp, vp, vp, i64, i64, ci, ci, vp], ci),
        "nhp_gated_act_bwd": ([vp, vp, vp, vp, i64, i64, ci, ci, vp], ci),
        "nhp_layernorm_fwd": ([vp, vp, vp, vp, vp, vp, f32, i64, i64, ci, ci, vp], ci),
        "nhp_layernorm_bwd": ([vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, ci, ci, vp], ci),
        "nhp_rmsnorm_fwd": ([vp, vp, vp, vp, vp, f32, ci, i64, i64, ci, ci, vp], ci),
        "nhp_rmsnorm_bwd": ([vp, vp, vp, vp, vp, vp, vp, vp, f32, ci, i64, i64, ci, ci, vp], ci),
        "nhp_layernorm_pair_fwd": ([vp, vp, vp, vp, vp, vp, vp, vp, vp, f32, i64, i64, ci, ci, vp], ci),
        "nhp_layernorm_pair_bwd": ([vp] * 13 + [i64, i64, ci, ci, vp], ci),
        "nhp_layernorm_pair_bwd_workspace_bytes": ([i64, i64, ci], i64),
        "nhp_column_sum": ([vp, vp, vp, i64, i64, ci, vp], ci),
        "nhp_column_sum_workspace_bytes": ([i64, i64, ci], i64),
        "nhp_rmsnorm_partial_fwd": ([vp, vp, vp, vp, vp, f32, ci, i64, i64, i64, ci, ci, vp], ci),
        "nhp_rmsnorm_partial_bwd": ([vp, vp, vp, vp, vp, vp, vp, vp, f32, ci, i64, i64, i64, ci, ci, vp], ci),
        "nhp_norm_bwd_workspace_bytes": ([i64, i64, ci], i64),
        "nhp_layernorm_bwd_noalloc": ([vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, ci, ci, vp], ci),
    }
    for name, (args, res) in sigs.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.argtypes = args
        fn.restype = res
    return sigs


EXPORTS = None


def lib():
    """The loaded library; raises ImportError when it is absent or stale."""
    global _lib, EXPORTS
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise ImportError(
                        f"{LIB_PATH} not found: the fused kernels are not built. "
                        "Run `from megatron.fused_kernels import load; load()`."
                    )
                try:
                    handle = ctypes.CDLL(LIB_PATH)
                    EXPORTS = _declare(handle)
                except (OSError, AttributeError) as e:
                    raise ImportError(f"cannot load {LIB_PATH}: {e}") from e
                if handle.nhp_abi_version() != ABI_VERSION:
                    raise ImportError(
                        f"{LIB_PATH} has ABI version {handle.nhp_abi_version()}, expected {ABI_VERSION}; rebuild it"
                    )
                _lib = handle
    return _lib


def check(status, what):
    if status != 0:
        msg = lib().nhp_status_string(status).decode()
        raise RuntimeError(f"{what}: {msg} (status {status})")


def dtype_code(t, what):
    try:
        return _DTYPE[t.dtype]
    except KeyError:
        raise RuntimeError(f"{what}: unsupported dtype {t.dtype}") from None


def forward_scale(scale_factor, t, narrow):
    """The factor the forward softmax kernels multiply the scores by. With ``narrow`` it is first rounded
    to t's dtype (round to nearest even) and widened again, which is what the reference's CUDA dispatchers do
    by taking ``const input_t scale`` (scaled_upper_triang_masked_softmax.h:368, scaled_masked_softmax.h:358);
    without it the fp32 value is used as it is, like the reference's backward and its torch branch."""
    value = float(scale_factor)
    if narrow:
        value = float(torch.tensor(value, dtype=torch.float32).to(t.dtype))
    return value


def require_gpu(t, what):
    if t.device.type != "cuda":
        raise RuntimeError(f"{what}: expected a tensor on the GPU, got device {t.device}")


# torch's direct accessor of the current stream's handle (what its own launchers use): about a microsecond
# less per call than building a torch.cuda.Stream object first
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(t):
    """The HIP stream torch would launch on for t's device right now, as a handle for the C ABI."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(t.device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


class _NoGuard:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(t):
    """Context manager that makes t's device current for the launch; free when it already is."""
    if t.device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(t.device)


def strides4(t):
    return (ctypes.c_int64 * 4)(*t.stride())
