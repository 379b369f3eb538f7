"""ctypes binding of ``libpariskv_hip.so`` (the C ABI in ``include/pariskv_hip.h``).

The library is the product's only compute path: there is no CPU or torch
fallback.  If it has not been built, loading raises with the build command.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# PARISKV_HIP_SO names another build of the library (same ABI), e.g. one compiled with different flags
SO_PATH = os.environ.get("PARISKV_HIP_SO") or os.path.join(_HERE, "libpariskv_hip.so")
CSRC = os.path.join(_HERE, "csrc")

OK, EINVAL, ENOMEM, EHIP = 0, -22, -12, -5
DTYPE_F32, DTYPE_BF16 = 0, 1
MAX_TIERS = 8

_vp, _i, _i64, _sz = C.c_void_p, C.c_int, C.c_int64, C.c_size_t


class AttnSegment(C.Structure):
    """Mirror of ``pkv_attn_segment``."""

    _fields_ = [("k", _vp), ("v", _vp), ("stride_b", _i64), ("stride_h", _i64), ("row0", _i64), ("n_rows", _i64),
                ("idx", _vp), ("idx_stride", _i64), ("idx_limit", _i64)]


class AttnArgs(C.Structure):
    """Mirror of ``pkv_attn_args``."""

    _fields_ = [("segments", AttnSegment * 4), ("n_segments", _i), ("row_keys", _vp), ("scale", C.c_float),
                ("out", _vp), ("ws", _vp), ("ws_bytes", _sz)]


class KvAppend(C.Structure):
    """Mirror of ``pkv_kv_append``."""

    _fields_ = [("dst_k", _vp), ("dst_v", _vp), ("stride_b", _i64), ("stride_h", _i64), ("rows", _i64), ("slot", _i64)]


class RetrieveArgs(C.Structure):
    """Mirror of ``pkv_retrieve_args``."""

    _fields_ = [
        ("q", _vp), ("dtype", _i), ("bs", _i), ("n_kv_heads", _i), ("group", _i),
        ("signs", _vp), ("centers", _vp), ("cluster_counts", _vp),
        ("codes", _vp), ("nib", _vp), ("weight", _vp),
        ("cap", _i64), ("key0", _i64), ("n_keys", _i64),
        ("tier_counts", C.c_uint32 * MAX_TIERS), ("n_tiers", _i),
        ("n_cand", _i64), ("k", _i64),
        ("out_ids", _vp), ("out_scores", _vp),
        ("src_k", _vp), ("src_v", _vp), ("gather_from_host", _i),
        ("src_len", _i64), ("idx_offset", _i64),
        ("dst_k", _vp), ("dst_v", _vp), ("dst_len", _i64), ("dst_row0", _i64),
        ("row_bytes", _i), ("any_order", _i), ("nib_key_stride", _i64), ("weight_key_stride", _i64),
        ("record_word_offset", _i64), ("launch_plan", _i), ("skip_vote_counts", _i), ("table_ready", _i),
    ]


PLAN_SEPARATE, PLAN_ONE_LAUNCH = 0, 1  # pkv_retrieve_args.launch_plan


class AdaptiveArgs(C.Structure):
    """Mirror of ``pkv_adaptive_args``."""

    _fields_ = [
        ("dense_k", _vp), ("dense_stride_b", _i64), ("dense_stride_h", _i64), ("dense_rows", _i64),
        ("dense_vnorm", _vp), ("dense_vnorm_stride", _i64), ("dense_logits", _vp), ("dense_logits_stride", _i64),
        ("scale", C.c_float), ("value_norm", _vp), ("vn_stride", _i64), ("vn_offset", _i64), ("vn_pos_stride", _i64),
        ("threshold", C.c_float), ("k_out", _i64), ("k_min", _i64), ("k_max", _i64),
        ("adaptive_k", _vp), ("topk_ids", _vp), ("row_keys", _vp), ("row_keys_base", _i64),
        ("uniform_k", _vp), ("ws", _vp), ("ws_bytes", _sz),
        ("src_k", _vp), ("src_v", _vp), ("src_len", _i64), ("idx_offset", _i64),
        ("dst_k", _vp), ("dst_v", _vp), ("dst_len", _i64), ("dst_row0", _i64), ("row_bytes", _i),
    ]


# name -> (restype, argtypes); one entry per declaration in include/pariskv_hip.h
PROTOTYPES = {
    "pkv_version": (_i, []),
    "pkv_last_error": (C.c_char_p, []),
    "pkv_struct_bytes": (_sz, [_i]),
    "pkv_encode_append": (_i, [_vp, _i, _i, _i, _i64, _i64, _i64, _i64, _vp,
                               _vp, _i64, _i64, _i64, _i64,
                               _vp, _i64, _i64, _i64, _i64,
                               _vp, _i64, _i64, _i64, _i64,
                               _vp, _i64, _i64, _vp]),
    "pkv_count_cluster_keys": (_i, [_vp, _i64, _i64, _i64, _i64, _i, _i, _i64, _vp, _i64, _i64, _vp]),
    "pkv_query_prep_lut": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _i64, _i64, _vp, _i, _vp, _vp, _vp, _vp, _vp]),
    "pkv_update_cache_cnt": (_i, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64,
                                  _i, _i, _i64, _vp, _i, _vp, _vp, _vp]),
    "pkv_update_cache_cnt_legacy": (_i, [_vp, _vp, _vp, _i, _i, _i64, _vp, _vp, _vp]),
    "pkv_collision_scan": (_i, [_vp, _i64, _i64, _i64, _i64, _i, _i, _i64, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "pkv_collision_scan_timed": (_i, [_vp, _i64, _i64, _i64, _i64, _i, _i, _i64, _vp, _vp, _i64, _vp, _vp, _i,
                                      C.POINTER(C.c_float), _vp]),
    "pkv_copy_bytes": (_i, [_vp, _vp, _sz, _vp]),
    "pkv_read_bytes": (_i, [_vp, _sz, _vp, _vp]),
    "pkv_bucket_topk_ws_bytes": (_sz, [_i, _i64]),
    "pkv_bucket_topk": (_i, [_vp, _i64, _i, _i64, _i64, _vp, _vp, _sz, _vp]),
    "pkv_topk_f32_ws_bytes": (_sz, [_i, _i64, _i64]),
    "pkv_topk_f32": (_i, [_vp, _i64, _vp, _i64, _i, _i64, _i64, _vp, _vp, _vp, _sz, _vp]),
    "pkv_rerank4": (_i, [_vp, _i, _i, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64,
                         _vp, _vp, _vp, _vp, _vp, _vp]),
    "pkv_gather_uva": (_i, [_vp, _vp, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i, _i, _i, _vp]),
    "pkv_gather_hbm": (_i, [_vp, _vp, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i, _i, _i, _vp]),
    "pkv_append_kv": (_i, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i, _i, _i,
                           _vp, _i64, _i64, _vp]),
    "pkv_offload_rows": (_i, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i, _i, _i, _vp]),
    "pkv_offload_rows_dma": (_i, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i, _i, _i, _i, _vp]),
    "pkv_gather_uva_ragged": (_i, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i64, _i64, _i, _i, _i, _vp]),
    "pkv_gather_uva_packed": (_i, [_vp, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "pkv_gather_cpu": (_i, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i, _i]),
    "pkv_host_alloc_mapped": (_i, [_sz, C.POINTER(_vp)]),
    "pkv_host_free": (_i, [_vp]),
    "pkv_host_device_pointer": (_i, [_vp, C.POINTER(_vp)]),
    "pkv_adaptive_topk_ws_bytes": (_sz, [_i, _i64, _i64]),
    "pkv_adaptive_topk": (_i, [_vp, _i64, _vp, _i64, _i64, _vp, _i, C.c_float, _vp, _vp, _i64, _i64, _i64, _vp, _i64,
                               C.c_float, _i64, _i, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _sz, _vp]),
    "pkv_uniform_k": (_i, [_vp, _i, _vp, _vp, _i64, _vp]),
    "pkv_dense_logits": (_i, [_vp, _i, _i, _i, _i, _vp, _i64, _i64, _i64, C.c_float, _vp, _i64, _vp]),
    "pkv_decode_attention_ws_bytes": (_sz, [_i, _i, _i, _i64]),
    "pkv_decode_attention": (_i, [_vp, _i, _i, _i, _i, C.POINTER(AttnSegment), _i, _vp, C.c_float, _vp, _vp, _sz, _vp]),
    "pkv_qk_norm_rope": (_i, [_vp, _i64, _i, _i, _i, _vp, _vp, C.c_float, _vp, _vp, _vp, _vp, _vp]),
    "pkv_add_rmsnorm": (_i, [_vp, _vp, _vp, C.c_float, _i, _i, _vp, _vp, _vp]),
    "pkv_silu_mul": (_i, [_vp, _i64, _i, _i, _vp, _vp]),
    "pkv_retrieve_ws_bytes": (_sz, [_i, _i64, _i64, _i64]),
    "pkv_retrieve": (_i, [C.POINTER(RetrieveArgs), _vp, _sz, _vp]),
    "pkv_qk_norm_rope_table": (_i, [_vp, _i64, _i, _vp, _vp, C.c_float, _vp, _vp, _vp, _vp, C.POINTER(RetrieveArgs), _vp, _sz,
                                    C.POINTER(KvAppend), _vp]),
    "pkv_retrieve_noalloc_max_bytes": (_sz, []),
    "pkv_retrieve_noalloc_prepare": (_i, []),
    "pkv_retrieve_noalloc": (_i, [C.POINTER(RetrieveArgs), _vp]),
    "pkv_decode_step": (_i, [C.POINTER(RetrieveArgs), _vp, _sz, C.POINTER(AttnArgs), _vp]),
    "pkv_adaptive_decode_step": (_i, [C.POINTER(RetrieveArgs), _vp, _sz, C.POINTER(AdaptiveArgs), C.POINTER(AttnArgs), _vp]),
    "pkv_retrieve_ws_view": (_i, [_vp, _i, _i64, _i64, _i64, C.c_char_p, C.POINTER(_vp), C.POINTER(_sz)]),
}


def build(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 into ``libpariskv_hip.so`` (always recompiles)."""
    cmd = ["make", "-B", "-j8", "-C", CSRC]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0 or verbose:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libpariskv_hip.so failed (see output above)")
    return SO_PATH


_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise RuntimeError(
                f"{SO_PATH} is missing: the HIP extension is the only compute path. "
                f"Build it with `make -C {CSRC}` (or `python -c 'import __graft_entry__ as g; g.build()'`).")
        handle = C.CDLL(SO_PATH)
        for name, (res, args) in PROTOTYPES.items():
            if os.environ.get("PARISKV_HIP_SO") and not hasattr(handle, name):
                continue  # optional symbols: an older build named by PARISKV_HIP_SO may lack the newest entry points
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        for which, mirror in enumerate((AttnSegment, AttnArgs, RetrieveArgs, AdaptiveArgs)):
            if handle.pkv_struct_bytes(which) != C.sizeof(mirror):
                raise RuntimeError(f"{SO_PATH} was built from another header: {mirror.__name__} is "
                                   f"{handle.pkv_struct_bytes(which)} bytes there, {C.sizeof(mirror)} here; rebuild it")
        _lib = handle
    return _lib


def check(rc: int) -> None:
    """Turn a negative return code into RuntimeError (the reference raises through TORCH_CHECK)."""
    if rc != OK:
        msg = lib().pkv_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"pariskv_hip error {rc}: {msg}")
