"""The C-ABI library loads on a machine without a GPU and exports every symbol the header declares; the pieces of
host logic that need no device (argument checks, size queries, libm calibration) behave.  (CPU only: no compute.)"""
import ctypes
import os
import re

import numpy as np
import pytest

import oracle
from nnabla_amd import kernels

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    names = set()
    inc = os.path.join(ROOT, "include")
    for f in os.listdir(inc):
        if f.endswith(".h"):
            text = open(os.path.join(inc, f)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names |= set(re.findall(r"\b(nbla_hip_[a-z0-9_]+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    L = kernels.lib()
    declared = _declared_symbols()
    assert declared, "no declarations found in include/*.h"
    missing = sorted(s for s in declared if not hasattr(L, s))
    assert not missing, "declared in include/ but not exported: %s" % missing
    assert declared == set(kernels.EXPORTED), sorted(declared ^ set(kernels.EXPORTED))
    assert b"gfx950" in L.nbla_hip_version()


def test_argument_errors_mirror_the_reference_checks():
    L = kernels.lib()
    null = ctypes.c_void_p(0)
    # fixed_point_quantize.cpp:31-32 and :41-42
    for sign, n, delta in [(1, 0, 0.1), (1, 8, 0.0), (1, 1, 0.1)]:
        assert L.nbla_hip_fixed_point_quantize_f32(null, null, ctypes.c_size_t(0), sign, n, ctypes.c_float(delta),
                                                   null) == kernels.ERR_VALUE
    assert b"bit width" in L.nbla_hip_last_error()
    # pow2_quantize.cpp:32 and :41-44
    for sign, wz, n in [(1, 1, 0), (1, 1, 2), (0, 1, 1)]:
        assert L.nbla_hip_pow2_quantize_f32(null, null, ctypes.c_size_t(0), sign, wz, n, 1, null) == kernels.ERR_VALUE
    # min_max_quantize.cpp:69-81: q shape must be 1 or equal to x's
    xs, qs = (ctypes.c_int64 * 2)(4, 6), (ctypes.c_int64 * 2)(1, 3)
    rc = L.nbla_hip_min_max_quantize_f32(null, null, xs, 2, qs, null, null, null, null, null, ctypes.c_float(0.9), 0,
                                         0, ctypes.c_float(0.01), null, ctypes.c_size_t(0), null)
    assert rc == kernels.ERR_VALUE


def test_size_queries():
    L = kernels.lib()
    i64 = ctypes.c_int64
    assert L.nbla_hip_packed_bits_bytes(i64(4096), i64(11008)) == 4096 * 11008 // 8
    assert L.nbla_hip_packed_bits_bytes(i64(33), i64(65)) == 8 * 1 * 64 * 16          # padded to 256 x 256
    # int8 digit operand: 3 bytes per element (K padded to 256), then per row one int64 sum per 16384-column chunk
    # and one int32 shift
    assert L.nbla_hip_digit_operand_bytes(i64(4096), i64(4096)) == 4096 * 4096 * 3 + 4096 * 12 + 256
    assert L.nbla_hip_digit_operand_bytes(i64(1), i64(1)) == 32 * 256 * 3 + 32 * 12 + 256
    assert L.nbla_hip_digit_operand_bytes(i64(32), i64(16385)) == 32 * 16640 * 3 + 32 * (2 * 8 + 4) + 256
    assert L.nbla_hip_binary_affine_workspace_bytes(i64(64), i64(256), i64(256)) % 256 == 0


@pytest.mark.parametrize("which,fn", [(0, oracle.round_log2), (1, oracle.inq_exponent), (2, oracle.inq_n1)])
def test_cut_tables_reproduce_host_libm(which, fn):
    """E + (bits >= cut[binade]) must equal the libm-based decision for every value near every cut, at the ends of
    every binade and on random values."""
    table = kernels.cut_table(which)
    assert len(table) == 277
    rng = np.random.RandomState(which)

    def binade(u):
        e = u >> 23
        return e + 22 if e else int(u).bit_length() - 1

    def check(u):
        u = int(u)
        if u == 0 or u >= 0x7f800000:
            return
        a = np.array([u], np.uint32).view(np.float32)[0]
        idx = binade(u)
        assert (idx - 149) + (1 if u >= table[idx] else 0) == fn(float(a)), (hex(u), idx)

    for idx in range(277):
        lo = (1 << idx) if idx < 23 else ((idx - 22) << 23)
        hi = ((1 << (idx + 1)) - 1) if idx < 23 else (lo | 0x7fffff)
        for u in (lo, hi, lo + 1, hi - 1):
            check(u)
        for d in range(-6, 7):
            check(min(max(table[idx] + d, lo), hi))
    for u in rng.randint(1, 0x7f800000, size=20000, dtype=np.int64):
        check(u)
