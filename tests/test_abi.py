"""CPU-only checks of the C-ABI boundary: the library loads, exports exactly what
include/pariskv_hip.h declares, and the Python binding has a prototype for each."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pariskv_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pkv_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("pkv_encode_append", "pkv_query_prep_lut", "pkv_update_cache_cnt", "pkv_bucket_topk", "pkv_topk_f32",
                 "pkv_rerank4", "pkv_gather_uva", "pkv_gather_hbm", "pkv_gather_cpu", "pkv_retrieve"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from pariskv_amd import _lib

    if not os.path.exists(_lib.SO_PATH):
        _lib.build()
    handle = ctypes.CDLL(_lib.SO_PATH)
    for name in declared_functions():
        assert hasattr(handle, name), f"{name} declared in the header but not exported"
        assert name in _lib.PROTOTYPES, f"{name} has no ctypes prototype"
    assert sorted(_lib.PROTOTYPES) == declared_functions()
    assert _lib.lib().pkv_version() >= 1


def test_every_declaration_cites_the_reference():
    text = open(HEADER).read()
    # each documented entry point names a reference file:line (or says it has no counterpart)
    blocks = re.findall(r"/\*(.*?)\*/\s*(?:size_t|int)\s+(pkv_[a-z0-9_]+)\s*\(", text, flags=re.S)
    assert len(blocks) >= 15
    for comment, name in blocks:
        assert re.search(r"\.(cu|py|cpp):\d+", comment) or "no counterpart" in comment.lower() or name in (
            "pkv_host_free", "pkv_host_device_pointer", "pkv_retrieve_ws_view"), name


def test_host_side_argument_errors_without_gpu():
    """Pure host validation paths return error codes and messages (no kernel is launched)."""
    from pariskv_amd import _lib

    L = _lib.lib()
    assert L.pkv_bucket_topk(None, 0, 1, 10, 5, None, None, 0, None) == _lib.EINVAL
    assert b"null pointer" in L.pkv_last_error()
    assert L.pkv_retrieve(None, None, 0, None) == _lib.EINVAL
    assert L.pkv_retrieve_ws_bytes(32, 131072, 4096, 1024) > 32 * 131072
    assert L.pkv_retrieve_ws_bytes(32, 100, 200, 10) == 0  # n_cand > n_keys
    with pytest.raises(RuntimeError, match="pariskv_hip error"):
        _lib.check(L.pkv_gather_cpu(None, None, None, None, None, 1, 1, 1, 1, 1, 2, 1))
    assert L.pkv_adaptive_decode_step(None, None, 0, None, None, None) == _lib.EINVAL
    a, ad, aa = _lib.RetrieveArgs(), _lib.AdaptiveArgs(), _lib.AttnArgs()
    a.out_ids = 8  # a final top-k was asked for: not the candidates-only form
    assert L.pkv_adaptive_decode_step(a, None, 0, ad, aa, None) == _lib.EINVAL
    assert b"candidates-only" in L.pkv_last_error()
    assert L.pkv_dense_logits(None, 1, 1, 1, 1, None, 0, 0, 1, 1.0, None, 1, None) == _lib.EINVAL
    assert L.pkv_adaptive_topk(None, 0, None, 0, 0, None, 0, 1.0, None, None, 0, 0, 0, None, 10, 0.9, 5, 1, None, None,
                               6, 5, None, 0, None, 0, None) == _lib.EINVAL
    assert b"clamp" in L.pkv_last_error()


def test_struct_mirrors_have_the_library_sizes():
    from pariskv_amd import _lib

    L = _lib.lib()
    for which, mirror in enumerate((_lib.AttnSegment, _lib.AttnArgs, _lib.RetrieveArgs, _lib.AdaptiveArgs)):
        assert L.pkv_struct_bytes(which) == ctypes.sizeof(mirror) > 0
    assert L.pkv_struct_bytes(4) == 0


def test_gather_cpu_host_function():
    """pkv_gather_cpu is host code: exercised fully on the CPU (gather_cpu.cpp contract)."""
    import torch

    from pariskv_amd.cache_hub.gather import load_gather_ext

    ext = load_gather_ext()
    g = torch.Generator().manual_seed(0)
    src = torch.randn(2, 3, 50, 128, generator=g).to(torch.bfloat16)
    idx = torch.randint(0, 50, (2, 3, 7), generator=g)
    out = torch.empty(2, 3, 7, 128, dtype=torch.bfloat16)
    ext.gather_kv_out_cpu(src, idx, out)
    assert torch.equal(out, torch.gather(src, 2, idx.unsqueeze(-1).expand(-1, -1, -1, 128)))
    src_t = torch.randn(2, 3, 128, 50, generator=g).transpose(2, 3)  # non-contiguous rows
    out32 = torch.empty(2, 3, 7, 128)
    ext.gather_kv_out_cpu(src_t, idx, out32)
    assert torch.equal(out32, torch.gather(src_t, 2, idx.unsqueeze(-1).expand(-1, -1, -1, 128)))
    idx[0, 0, 0] = 50
    with pytest.raises(RuntimeError, match="out of bounds"):
        ext.gather_kv_out_cpu(src, idx, out)


def test_gather_cpu_equals_the_reference_build():
    """pkv_gather_cpu and the oracle's gather_rows against the reference's own gather_cpu.cpp, compiled by
    oracle/build_ref.py into oracle/_ref (skipped where that build is absent)."""
    import numpy as np
    import torch

    from oracle import build_ref
    from oracle import pkv_oracle as O
    from pariskv_amd.cache_hub.gather import load_gather_ext

    ref = build_ref.load()
    if ref is None:
        pytest.skip("oracle/_ref is not built (python oracle/build_ref.py needs the reference tree)")
    ext = load_gather_ext()
    g = torch.Generator().manual_seed(3)
    for dtype, shape, K in ((torch.bfloat16, (2, 8, 3000, 128), 100), (torch.float32, (1, 3, 77, 128), 77),
                            (torch.float16, (3, 2, 500, 64), 1)):
        src = torch.randn(*shape, generator=g).to(dtype)
        idx = torch.randint(0, shape[2], (shape[0], shape[1], K), generator=g)
        want = torch.empty(shape[0], shape[1], K, shape[3], dtype=dtype)
        got = torch.full_like(want, 7)
        ref.gather_kv_out_cpu(src, idx, want)
        ext.gather_kv_out_cpu(src, idx, got)
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))
        for b in range(shape[0]):
            for h in range(shape[1]):
                rows = O.gather_rows(src[b, h].view(torch.uint8).numpy(), idx[b, h].numpy())
                assert np.array_equal(rows, want[b, h].view(torch.uint8).numpy())
    # rows that are not contiguous, and an output that is a slice of a larger buffer
    src_t = torch.randn(2, 3, 128, 50, generator=g).transpose(2, 3)
    idx = torch.randint(0, 50, (2, 3, 9), generator=g)
    big_w, big_g = torch.zeros(2, 3, 20, 128), torch.zeros(2, 3, 20, 128)
    ref.gather_kv_out_cpu(src_t, idx, big_w[:, :, 4:13])
    ext.gather_kv_out_cpu(src_t, idx, big_g[:, :, 4:13])
    assert torch.equal(big_g, big_w)
    idx[1, 2, 8] = -1
    with pytest.raises(RuntimeError, match="out of bounds"):
        ref.gather_kv_out_cpu(src_t, idx, big_w[:, :, 4:13])
    with pytest.raises(RuntimeError, match="out of bounds"):
        ext.gather_kv_out_cpu(src_t, idx, big_g[:, :, 4:13])
