"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol
and rejects bad arguments before anything reaches a GPU."""
import ctypes
import os
import re

from blockedattention_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "blocked_attention.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ba_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert declared_symbols() == sorted(capi.SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    for name in declared_symbols():
        assert hasattr(lib, name), name
    assert lib.ba_abi_version() == 5


def test_plan_bytes_and_status_strings():
    lib = capi.load()
    sizes = [lib.ba_plan_bytes(n) for n in (0, 1, 64, 1024, 100000)]
    assert all(s % 256 == 0 and s > 0 for s in sizes) and sizes == sorted(sizes)
    assert lib.ba_plan_bytes(-1) == 0
    assert lib.ba_status_string(0) == b"ok"
    assert len({lib.ba_status_string(i) for i in range(6)}) == 6


def test_argument_errors_are_reported_without_a_device():
    lib = capi.load()
    null = ctypes.c_void_p(0)
    assert lib.ba_plan_gemm(null, 0, 4, 0, null, null, null, null, null, null, null) == 1       # no plan buffer
    buf = (ctypes.c_char * 65536)()
    p = ctypes.c_void_p((ctypes.addressof(buf) + 255) & ~255)
    assert lib.ba_plan_gemm(p, 16, 4, 0, null, null, null, null, null, null, null) == 2          # buffer too small
    assert lib.ba_plan_gemm(p, 60000, 4, 7, null, null, null, null, null, null, null) == 1       # unknown mode
    assert lib.ba_plan_gemm(p, 60000, 4, 0, null, null, null, null, null, null, null) == 1       # lists missing
    assert lib.ba_plan_gemm(p, 60000, -1, 0, null, null, null, null, null, null, null) == 1      # negative count
    assert lib.ba_plan_read(null, None, null) == 1
    assert lib.ba_varlen_gemm(null, None, 1, 0, null, null, null, 1, 1, 1, 1, 0, 0, null) == 1
    assert lib.ba_varlen_gemm(p, None, 1, 0, null, null, null, -1, 1, 1, 1, 0, 0, null) == 1
    assert lib.ba_gemm_softmax(p, None, 1, 2, p, p, p, 2, 1, 8, 8, 1, 1.0, null) == 3                # fp32 operands
    assert lib.ba_gemm_softmax(p, None, 1, 0, p, p, p, 1, 1, 8, 8, 1, 1.0, null) == 3                # f16 in, bf16 out
    assert lib.ba_blocked_softmax(null, None, 1, 0, null, null, 1, 1, 1.0, null) == 1
    assert lib.ba_varlen_attention(p, None, 1, 2, p, p, p, p, 1, 8, 8, 1, 1.0, null) == 3            # fp32 operands
    assert lib.ba_varlen_attention(p, None, 1, 0, p, p, null, p, 1, 8, 8, 1, 1.0, null) == 1         # no values
    assert lib.ba_varlen_attention(null, None, 1, 0, p, p, p, p, 1, 8, 8, 1, 1.0, null) == 1         # no plan
    assert lib.ba_varlen_attention(p, None, 0, 0, p, p, p, p, 1, 8, 8, 1, 1.0, null) == 0            # no segments
    # empty work is not an error and launches nothing
    assert lib.ba_varlen_gemm(p, None, 1, 0, null, null, null, 0, 0, 0, 0, 0, 0, null) == 0
    assert lib.ba_blocked_softmax(p, None, 1, 0, null, null, 4, 0, 1.0, null) == 0
