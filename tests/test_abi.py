"""CPU-only checks of the C ABI: the library loads, exports every symbol the header declares, the
Python mirror of the params struct has the library's size, and the pure host functions agree with
the oracle.  No kernel is launched."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fa_mi355x.h")
LIB = os.path.join(ROOT, "flash-attention_amd", "flash_attn", "libfa_mi355x.so")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        import __graft_entry__
        __graft_entry__.build()
    return ctypes.CDLL(LIB)


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fa_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_exported(lib):
    names = declared_symbols()
    assert {"fa_fwd", "fa_varlen_fwd", "fa_fwd_kvcache", "fa_plan_splits", "fa_last_error",
            "fa_num_splits_heuristic_reference", "fa_version", "fa_sizeof_params", "fa_bwd", "fa_varlen_bwd",
            "fa_sizeof_bwd_params", "fa_rotary", "fa_sizeof_rotary_params"} <= set(names)
    for n in names:
        assert hasattr(lib, n), "library does not export %s" % n


def test_kernel_ids_of_the_header_have_names():
    """Every FA_KERNEL_* id that fa_last_kernel() can return is decoded by flash_attn._native.last_kernel()."""
    import flash_attn._native as nat
    text = open(HEADER).read()
    ids = {name: int(val) for name, val in re.findall(r"#define\s+FA_KERNEL_((?!FLAG_)[A-Z0-9_]+)\s+(\d+)\b", text)}
    assert ids["NONE"] == 0 and len(ids) >= 10 and len(set(ids.values())) == len(ids)
    assert set(ids.values()) == set(nat.KERNEL_NAMES)
    for name, val in ids.items():
        assert nat.KERNEL_NAMES[val] == name.lower(), (name, val, nat.KERNEL_NAMES[val])


def test_struct_mirror_size(lib):
    import flash_attn._native as nat
    lib.fa_sizeof_params.restype = ctypes.c_int32
    assert lib.fa_sizeof_params() == ctypes.sizeof(nat.FaFwdParams)
    lib.fa_sizeof_bwd_params.restype = ctypes.c_int32
    assert lib.fa_sizeof_bwd_params() == ctypes.sizeof(nat.FaBwdParams)
    lib.fa_sizeof_rotary_params.restype = ctypes.c_int32
    assert lib.fa_sizeof_rotary_params() == ctypes.sizeof(nat.FaRotaryParams)


def test_backward_argument_errors_do_not_abort(lib):
    import flash_attn._native as nat
    p = nat.FaBwdParams()
    lib.fa_bwd.argtypes = [ctypes.POINTER(nat.FaBwdParams), ctypes.c_void_p]
    lib.fa_bwd.restype = ctypes.c_int
    lib.fa_varlen_bwd.argtypes = [ctypes.POINTER(nat.FaBwdParams), ctypes.c_void_p]
    lib.fa_varlen_bwd.restype = ctypes.c_int
    lib.fa_last_error.restype = ctypes.c_char_p
    assert lib.fa_bwd(ctypes.byref(p), None) != 0 and b"must be set" in lib.fa_last_error()
    for n in ("dout", "q", "k", "v", "out", "softmax_lse", "dq", "dk", "dv", "softmax_d"):
        setattr(p, n, 16)                       # never dereferenced: the checks below fail first
    p.b, p.h, p.h_k, p.d, p.seqlen_q, p.seqlen_k, p.seqlen_q_rounded, p.dtype = 1, 4, 3, 64, 8, 8, 128, 1
    assert lib.fa_bwd(ctypes.byref(p), None) != 0 and b"Number of heads" in lib.fa_last_error()
    p.h_k, p.d = 2, 260
    assert lib.fa_bwd(ctypes.byref(p), None) != 0 and b"at most 256" in lib.fa_last_error()
    p.d = 64
    assert lib.fa_varlen_bwd(ctypes.byref(p), None) != 0 and b"cu_seqlens" in lib.fa_last_error()
    p.q_row_stride = 4
    assert lib.fa_bwd(ctypes.byref(p), None) != 0 and b"strides" in lib.fa_last_error()
    p.q_row_stride, p.dk_row_stride = 0, 4     # gradients leave 16 bytes per lane as well
    assert lib.fa_bwd(ctypes.byref(p), None) != 0 and b"strides" in lib.fa_last_error()
    p.dk_row_stride, p.dv = 0, 24
    assert lib.fa_bwd(ctypes.byref(p), None) != 0 and b"16-byte aligned" in lib.fa_last_error()
    p.dv, p.p_dropout = 16, 0.1
    assert lib.fa_bwd(ctypes.byref(p), None) != 0 and b"rng_state" in lib.fa_last_error()
    p.p_dropout = 1.0
    assert lib.fa_bwd(ctypes.byref(p), None) != 0 and b"p_dropout" in lib.fa_last_error()


def test_reference_heuristic_matches_oracle(lib):
    from oracle import attention_oracle as orc
    f = lib.fa_num_splits_heuristic_reference
    f.argtypes = [ctypes.c_int32] * 4
    f.restype = ctypes.c_int
    assert f(48, 108, 64, 128) == 2       # csrc/flash_attn/flash_api.cpp:206-211
    for blocks in (1, 2, 5, 13, 48, 80, 87, 200):
        for sms in (80, 108, 132, 256):
            for nb in (1, 2, 7, 64, 257):
                assert f(blocks, sms, nb, 128) == orc.num_splits_heuristic_reference(blocks, sms, nb, 128)


def test_argument_errors_do_not_abort(lib):
    import flash_attn._native as nat
    p = nat.FaFwdParams()
    lib.fa_fwd.argtypes = [ctypes.POINTER(nat.FaFwdParams), ctypes.c_void_p]
    lib.fa_fwd.restype = ctypes.c_int
    lib.fa_last_error.restype = ctypes.c_char_p
    assert lib.fa_fwd(ctypes.byref(p), None) != 0
    assert lib.fa_last_error()
    n = ctypes.c_int32(0)
    lib.fa_plan_splits.argtypes = [ctypes.POINTER(nat.FaFwdParams), ctypes.c_int32, ctypes.POINTER(ctypes.c_int32)]
    p.q = p.k = p.v = p.o = p.softmax_lse = 16   # never dereferenced by the planner
    p.b, p.h, p.h_k, p.d, p.seqlen_q, p.seqlen_k, p.dtype = 64, 64, 8, 128, 1, 32768, 1
    assert lib.fa_plan_splits(ctypes.byref(p), 2, ctypes.byref(n)) == 0
    assert 1 < n.value <= 128
    p.num_splits = 1
    assert lib.fa_plan_splits(ctypes.byref(p), 2, ctypes.byref(n)) == 0 and n.value == 1
    p.d = 260
    assert lib.fa_plan_splits(ctypes.byref(p), 2, ctypes.byref(n)) != 0
