"""The C-ABI library loads and exports every symbol include/rmlx_hip.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "rmlx_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rmlx_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_bound_symbols():
    from rmlx_amd import runtime
    assert sorted(runtime.EXPORTS) == _declared()


def test_library_exports_every_declared_symbol():
    from rmlx_amd import runtime
    if not os.path.exists(runtime.LIB_PATH):
        pytest.fail(f"{runtime.LIB_PATH} not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
    lib = ctypes.CDLL(runtime.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name


def test_library_exports_nothing_else():
    """Hidden visibility plus a version script: the dynamic symbol table is exactly the header's functions."""
    import shutil
    import subprocess
    from rmlx_amd import runtime
    nm = shutil.which("nm") or "/opt/rocm/llvm/bin/llvm-nm"
    out = subprocess.run([nm, "-D", "--defined-only", runtime.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.strip())
    assert exported == _declared()


def test_calls_fail_loudly_without_a_gpu_context():
    """No CPU fallback: compute entry points refuse to run before rmlx_hip_init succeeded."""
    from rmlx_amd import runtime as rt
    L = rt.lib()
    if rt._initialised:
        pytest.skip("a GPU context already exists in this process")
    a = rt.RmlxArray()
    st = L.rmlx_hip_affine_quantized_matmul_batched(None, ctypes.byref(a), None, 0, None)
    assert st == rt.RUNTIME_ERROR
    assert b"rmlx_hip_init" in L.rmlx_hip_last_error()


def test_qweight_validation_needs_no_gpu():
    """`QuantizedWeight::new` rules (quantized.rs:97-160) are pure host logic."""
    from rmlx_amd import runtime as rt
    L = rt.lib()
    h = ctypes.c_void_p()
    fake = ctypes.c_void_p(0x1000)

    def create(wb, sb, bb, gs, bits, n, k, e=1):
        return L.rmlx_hip_qweight_create(fake, wb, fake, sb, fake, bb, gs, bits, n, k, e, ctypes.byref(h))

    assert create(8 * 64 // 2, 16, 16, 64, 4, 8, 64) == rt.OK
    L.rmlx_hip_qweight_destroy(h)
    for args, msg in [((256, 16, 16, 64, 5, 8, 64), b"unsupported bit width 5"),
                      ((256, 16, 16, 48, 4, 8, 64), b"unsupported group_size 48"),
                      ((256, 16, 16, 128, 4, 8, 64), b"must be a multiple of group_size"),
                      ((255, 16, 16, 64, 4, 8, 64), b"weights_buf too small"),
                      ((256, 15, 16, 64, 4, 8, 64), b"scales_buf too small"),
                      ((256, 16, 15, 64, 4, 8, 64), b"biases_buf too small")]:
        assert create(*args) == rt.INVALID_SHAPE
        assert msg in L.rmlx_hip_last_error(), (msg, L.rmlx_hip_last_error())
    # all five bit widths of the reference type are accepted (quantized.rs:64)
    for bits in (2, 3, 4, 6, 8):
        per = 32 // bits
        assert create(((8 * 64 + per - 1) // per) * 4, 16, 16, 64, bits, 8, 64) == rt.OK
        L.rmlx_hip_qweight_destroy(h)


def test_expert_gemm_threshold_lives_in_the_handle():
    """The GEMV / grouped-GEMM threshold of the expert projections: default 10 rows per expert, per weight handle (no
    process-wide state), set returns the old value."""
    from rmlx_amd import runtime as rt
    L = rt.lib()
    hs = [ctypes.c_void_p(), ctypes.c_void_p()]
    for h in hs:
        assert L.rmlx_hip_qweight_create(ctypes.c_void_p(16), 1 << 20, ctypes.c_void_p(16), 1 << 20, ctypes.c_void_p(16), 1 << 20,
                                         64, 4, 64, 64, 2, ctypes.byref(h)) == rt.OK
    try:
        assert L.rmlx_hip_qweight_set_expert_gemm_min_rows(hs[0], 5) == 10
        assert L.rmlx_hip_qweight_set_expert_gemm_min_rows(hs[0], 0) == 5
        assert L.rmlx_hip_qweight_set_expert_gemm_min_rows(hs[1], 9) == 10  # the other handle kept its default
        assert L.rmlx_hip_qweight_set_expert_gemm_min_rows(hs[0], 10) == 0
    finally:
        for h in hs:
            L.rmlx_hip_qweight_destroy(h)
