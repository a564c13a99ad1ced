"""ctypes binding of libadamas_hip.so (see include/adamas_hip.h for the C ABI).

The library is loaded lazily and exactly once.  There is no fallback: if the shared object is missing
or an entry point fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint32, c_uint64, c_void_p
from pathlib import Path

import torch  # noqa: F401  (loads the HIP runtime this library binds to, before the library itself)

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libadamas_hip.so"

# name -> (restype, argtypes); order and types mirror include/adamas_hip.h
_SIGNATURES = {
    "adamas_version": (c_int, []),
    "adamas_error_string": (c_char_p, [c_int]),
    "adamas_hadamard": (c_int, [c_void_p, c_void_p, c_uint64, c_float, c_void_p]),
    "adamas_pack_2bit": (c_int, [c_void_p, c_void_p, c_uint64, c_void_p]),
    "adamas_append_decode": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32,
                                      c_uint32, c_uint32, c_uint32, c_float, c_uint32, c_void_p]),
    "adamas_append_prefill": (c_int, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p,
                                       c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32,
                                       c_float, c_uint32, c_void_p]),
    "adamas_estimate": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                 c_int64, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
                                 c_void_p]),
    "adamas_topk": (c_int, [c_void_p, c_int64, c_uint32, c_void_p, c_uint32, c_int32, c_void_p,
                             c_int64, c_uint32, c_uint32, c_void_p, c_void_p, c_int64, c_uint32,
                             c_void_p, c_size_t, c_void_p]),
    "adamas_read_probe": (c_int, [c_void_p, c_size_t, c_void_p, c_void_p]),
    "adamas_topk_workspace_bytes": (c_size_t, [c_uint32, c_uint32, c_uint32]),
    "adamas_workspace_bytes": (c_size_t, [c_uint32, c_uint32, c_uint32, c_uint32]),
    "adamas_sparse_decode": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int64, c_uint32, c_void_p, c_void_p, c_size_t, c_uint32,
                                      c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_uint32,
                                      c_void_p]),
    "adamas_decode_step": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_size_t,
                                    c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_float,
                                    c_uint32, c_uint32, c_void_p]),
    "adamas_step_fused_supported": (c_int, [c_uint32, c_uint32, c_uint32, c_uint32]),
    "adamas_step_plan": (c_int, [c_uint32, c_uint32, c_uint32, c_uint32, c_void_p]),
    "adamas_decode_step_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_uint32, c_void_p, c_void_p, c_uint32, c_uint32,
                                            c_uint32, c_uint32, c_uint32, c_float, c_uint32, c_uint32,
                                            c_uint32, c_void_p]),
    "adamas_step_candidates": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32,
                                        c_void_p, c_size_t, c_uint32, c_uint32, c_uint32, c_uint32,
                                        c_uint32, c_uint32, c_void_p]),
    "adamas_step_attend": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_uint32, c_void_p, c_void_p, c_void_p, c_size_t, c_uint32,
                                    c_uint32, c_uint32, c_uint32, c_uint32, c_float, c_uint32,
                                    c_uint32, c_void_p]),
    "adamas_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32,
                               c_float, c_void_p]),
    "adamas_rope_split": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_void_p,
                                   c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32,
                                   c_void_p]),
    "adamas_silu_mul": (c_int, [c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]),
    "adamas_rope_in_place": (c_int, [c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32,
                                      c_uint32, c_float, c_float, c_uint32, c_void_p]),
    "adamas_rope_append_decode": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32,
                                           c_uint32, c_uint32, c_uint32, c_float, c_uint32, c_void_p]),
    "adamas_decode_layer_step": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_uint32, c_void_p, c_void_p, c_void_p,
                                          c_size_t, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
                                          c_float, c_uint32, c_uint32, c_float, c_uint32, c_void_p]),
    "adamas_gemv": (c_int, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]),
    "adamas_gemv_silu_gate": (c_int, [c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]),
    "adamas_gemv_add": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]),
    "adamas_gemv_normed": (c_int, [c_void_p, c_void_p, c_void_p, c_uint32, c_float, c_void_p, c_uint32,
                                   c_uint32, c_void_p]),
    "adamas_gemv_silu_gate_normed": (c_int, [c_void_p, c_void_p, c_void_p, c_uint32, c_float, c_void_p,
                                             c_uint32, c_uint32, c_void_p]),
    "adamas_sumsq_partials": (c_int, [c_void_p, c_void_p, c_uint32, c_void_p]),
}

# entry points with a flags argument (include/adamas_hip.h): the prototype of the plain entry point
# with a uint32 `flags` inserted ahead of the stream
for _name in ("adamas_hadamard", "adamas_pack_2bit", "adamas_sparse_decode", "adamas_decode_step",
              "adamas_step_candidates", "adamas_step_attend"):
    _res, _args = _SIGNATURES[_name]
    _SIGNATURES[_name + "_f"] = (_res, _args[:-1] + [c_uint32, _args[-1]])

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

# constants of include/adamas_hip.h
F_CODE_FROM_FP32 = 1
F_BF16 = 2
F_HND = 4
F_NO_MFMA = 8
STATIC_SCRATCH_BYTES = 24 << 20
E_SCRATCH = -5
DIST_FP16, DIST_U16 = 0, 1
KEY_FP16_GENERIC, KEY_FP16_INT, KEY_U16_INT = 0, 1, 2

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library and attach the prototypes.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m adamas_amd.build` "
            "(there is no CPU or eager fallback for the Adamas HIP path)")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def step_plan(batch: int, num_heads: int, max_seq_len: int, budget: int) -> dict:
    """The geometry of the two-launch decode step for these sizes (adamas_step_plan)."""
    out = (c_uint32 * 8)()
    check(load().adamas_step_plan(batch, num_heads, max_seq_len, budget, ctypes.addressof(out)),
          "adamas_step_plan")
    keys = ("ok", "heads", "chunks", "units_q", "units_r", "passes", "partial", "kc")
    return dict(zip(keys, (int(v) for v in out)))


def error_string(code: int) -> str:
    return load().adamas_error_string(code).decode()


def check(code: int, what: str) -> None:
    """Raise RuntimeError for a non-zero return code, like TORCH_CHECK on a cudaError_t in the
    reference bindings (adamas/ops/csrc/page.cu:101-108)."""
    if code != 0:
        raise RuntimeError(f"{what} failed with error code {code}: {error_string(code)}")


def dtype_flags(dtype) -> int:
    """The `flags` bit of the append entry points for this dtype."""
    if dtype == torch.float16:
        return 0
    if dtype == torch.bfloat16:
        return F_BF16
    raise RuntimeError(f"only float16 and bfloat16 are supported, got {dtype}")


def ptr(t) -> int | None:
    """Device address of a tensor (None stays NULL)."""
    return None if t is None else t.data_ptr()


def current_stream() -> int:
    return torch.cuda.current_stream().cuda_stream
