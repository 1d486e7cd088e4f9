import ctypes
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs an AMD GPU (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session")
def c_oracle():
    """The scalar C restatement (oracle/nf4_ref.c) as a ctypes library; built on demand with gcc."""
    path = os.path.join(ROOT, "oracle", "_build", "libttamd_oracle.so")
    src = os.path.join(ROOT, "oracle", "nf4_ref.c")
    if not os.path.exists(path) or os.path.getmtime(path) < os.path.getmtime(src):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-B"], check=True, capture_output=True)
    lib = ctypes.CDLL(path)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.ref_nf4_quantize.argtypes = [vp, i32, i64, i32, i32, vp, vp, vp, vp, vp]
    lib.ref_nf4_quantize.restype = None
    lib.ref_nf4_dequantize.argtypes = [vp, vp, vp, vp, i32, i64, i32, i32, vp]
    lib.ref_nf4_dequantize.restype = None
    lib.ref_fq_per_token.argtypes = [vp, i32, i64, i64, vp, vp, vp]
    lib.ref_fq_per_token.restype = None
    lib.ref_fq_per_group.argtypes = [vp, i32, i64, i64, i32, vp, vp, vp]
    lib.ref_fq_per_group.restype = None
    lib.ref_fq_per_token_qp.argtypes = [vp, i32, i32, i64, i64, vp, vp, vp]
    lib.ref_fq_per_token_qp.restype = None
    lib.ref_fq_per_group_qp.argtypes = [vp, i32, i32, i64, i64, i32, vp, vp, vp]
    lib.ref_fq_per_group_qp.restype = None
    lib.ref_fq_per_group_uint4_asym.argtypes = [vp, i32, i32, i64, i64, i32, vp, vp, vp, vp]
    lib.ref_fq_per_group_uint4_asym.restype = None
    lib.ref_check_shared_reciprocal_division.argtypes = [i32, i32]
    lib.ref_check_shared_reciprocal_division.restype = i64
    lib.ref_check_code_table.argtypes = [vp]
    lib.ref_check_code_table.restype = i32
    return lib
