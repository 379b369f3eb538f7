"""Named host-side ranges for `rocprofv3 --marker-trace`, switched on with PARISKV_RANGES=1.

The reference brackets the decode step with NVTX ranges (`model_hub/LLM.py:173-183`: "decode_update_kv_cache",
"decode_attention"; `cache_hub/polar_cache_adaptivek_varlen.py:1483-1771`: "collision_based_topk_batch",
"adaptive_k0_pre", "compute_attention_varlen", ...).  On ROCm the same thing is a roctx range.  Here the whole
retrieval + gather + attention of a layer is ONE host call, so the ranges inside it collapse to one per call site; the
names say which of the reference's ranges each one covers.

Off (the default) a range costs one attribute test; on, two calls into the roctx library per range."""
import contextlib
import ctypes
import os

_push = _pop = None


def _load():
    global _push, _pop
    for name in ("librocprofiler-sdk-roctx.so", "libroctx64.so"):
        try:
            lib = ctypes.CDLL(name)
        except OSError:
            continue
        lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
        lib.roctxRangePushA.restype = ctypes.c_int
        lib.roctxRangePop.restype = ctypes.c_int
        _push, _pop = lib.roctxRangePushA, lib.roctxRangePop
        return True
    return False


enabled = os.environ.get("PARISKV_RANGES") == "1" and _load()


def push(name: str) -> None:
    if enabled:
        _push(name.encode())


def pop() -> None:
    if enabled:
        _pop()


@contextlib.contextmanager
def span(name: str):
    if enabled:
        _push(name.encode())
        try:
            yield
        finally:
            _pop()
    else:
        yield
