"""The C-ABI library loads and exports every symbol include/blr.h declares (no GPU work)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "mem-efficient-blr_amd", "lib", "libblr.so")
HDR = os.path.join(ROOT, "include", "blr.h")


def _declared():
    src = open(HDR).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(blr_[a-z0-9_]+)\s*\(", src)))


@pytest.fixture(scope="module")
def handle():
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} missing - run `python -c 'import __graft_entry__ as g; g.build()'`")
    return ctypes.CDLL(LIB)


def test_header_symbols_are_exported(handle):
    names = _declared()
    assert len(names) >= 14
    for n in names:
        assert hasattr(handle, n), f"{n} declared in blr.h but not exported"


def test_binding_table_matches_header():
    from triton_funcs import _lib
    assert _lib.exported_symbols() == _declared()


def test_argument_validation_needs_no_gpu(handle):
    handle.blr_last_error.restype = ctypes.c_char_p
    handle.blr_blast_workspace_bytes.restype = ctypes.c_size_t
    assert handle.blr_version() >= 100
    # tiled workspace = two (b, M, r) buffers of the dtype
    assert handle.blr_blast_workspace_bytes(2048, 4096, 4096, 16, 512, 0, 2) == 2 * 16 * 2048 * 512 * 2
    assert handle.blr_blast_workspace_bytes(0, 4096, 4096, 16, 512, 0, 2) == 0
    i64, vp = ctypes.c_int64, ctypes.c_void_p
    rc = handle.blr_dense_fwd(vp(0), i64(0), vp(0), vp(0), i64(0), 1, 1, 1, 0, 0, vp(0), ctypes.c_size_t(0), vp(0))
    assert rc == -1 and b"null" in handle.blr_last_error()
    rc = handle.blr_quantize_sym(vp(0), 0, i64(1), i64(1), i64(1), 8, vp(0), vp(0), vp(0))
    assert rc == -1


def test_shim_exports_reference_names():
    import importlib
    want = {
        "blast_kernels": ["triton_blast_partial_fp32", "triton_blast_partial_fp16", "triton_blast_partial_grouped_fp32",
                          "triton_blast_partial_grouped_fp16", "triton_blast_partial_grouped_persistent_fp32",
                          "triton_blast_partial_grouped_persistent_fp16", "triton_blast_full_fp32", "triton_blast_full_fp16",
                          "triton_blast_bmm_fp32", "triton_blast_bmm_fp16", "get_triton_blast_partial_fp16_config",
                          "get_triton_blast_partial_grouped_fp16_config", "get_triton_blast_partial_grouped_persistent_fp16_config",
                          "get_triton_blast_full_fp16_config", "get_triton_blast_bmm_xv_fp16_config",
                          "get_triton_blast_bmm_sxv_fp16_config", "get_triton_blast_bmm_usxv_fp16_config"],
        "blast_sym_quant_kernels": ["triton_blast_bmm_int8_fp16", "get_triton_blast_bmm_xv_int8_fp16_config",
                                    "get_triton_blast_bmm_sxv_int8_fp16_config", "get_triton_blast_bmm_usxv_int8_fp16_config"],
        "monarch_kernels": ["triton_monarch_right_fp32", "triton_monarch_right_fp16", "triton_monarch_right_ideal_fp32",
                            "triton_monarch_right_ideal_fp16", "triton_monarch_right_left_fp32", "triton_monarch_right_left_fp16",
                            "get_triton_monarch_right_fp16_config", "get_triton_monarch_right_ideal_fp16_config",
                            "get_triton_monarch_right_left_fp16_config"],
        "low_rank_kernels": ["triton_low_rank_fp32", "triton_low_rank_fp16", "triton_low_rank_load_store_fp32",
                             "triton_low_rank_load_store_fp16", "get_triton_low_rank_fp16_config"],
        "dense_kernels": ["triton_dense_fp32", "triton_dense_fp16", "triton_dense_load_store_fp32",
                          "triton_dense_load_store_fp16", "get_triton_dense_fp16_config"],
    }
    for mod, names in want.items():
        m = importlib.import_module(f"triton_funcs.{mod}")
        for n in names:
            assert callable(getattr(m, n)), f"triton_funcs.{mod}.{n} missing"


def test_no_cpu_fallback():
    """The product refuses CPU tensors instead of computing on the host."""
    import torch
    from triton_funcs import blast_kernels as K, _lib
    x = torch.zeros(1, 1, 4); U = torch.zeros(2, 2, 2); V = torch.zeros(2, 2, 2); S = torch.zeros(2, 2, 2)
    with pytest.raises(_lib.BlrError):
        K.triton_blast_full_fp32(x, U, V, S)


def test_run_time_options_are_named_and_range_checked():
    """blr_set_option knows every switch of the library by name and refuses values outside its range (no kernel launch is
    involved: the table lives on the host)."""
    from triton_funcs import _lib
    lib = _lib.lib()
    ok = {"BLR_GEMM_RING": (0, 1, 2), "BLR_GEMM_RING_TILE": (0, 256256, 256128, 256096, 128128), "BLR_GEMM_RING_PER_CU": (0, 1, 2),
          "BLR_GEMM_RING_WAVES": (4, 8), "BLR_GEMM_RING_BK": (32, 64), "BLR_GEMM_SPLITK": (0, 1), "BLR_DECODE2": (0, 1), "BLR_DECODE3": (0, 1),
          "BLR_DECODE_PAIR": (0, 1, 2), "BLR_DECODE_ROWS": (0, 1), "BLR_DENSE_SLAB": (0, 1), "BLR_DENSE_ROWS": (0, 1),
          "BLR_BLAST_MIXU": (0, 1, 2), "BLR_BLAST_ONE": (0, 1), "BLR_BLAST_YMIXW": (0, 1)}
    for name, values in ok.items():
        for v in values:
            assert lib.blr_set_option(name.encode(), v, 0) == 0, (name, v)
        for bad in (-1, 3, 100, 12345):
            if bad not in values:
                assert lib.blr_set_option(name.encode(), bad, 0) == -1, (name, bad)
                assert name.encode() in lib.blr_last_error()
        assert lib.blr_set_option(name.encode(), 0, 1) == 0            # back to "not set"
    assert lib.blr_set_option(b"BLR_NO_SUCH_SWITCH", 1, 0) == -1
