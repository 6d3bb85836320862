"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares,
answers capability questions without a device, and validates shapes before touching the GPU.
No kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import frink_amd as fa

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "frink_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(frk_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = fa.lib()
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(L, n), "libfrink_hip.so does not export %s" % n
    assert sorted(fa.EXPORTS) == names, "frink_amd.EXPORTS and include/frink_hip.h disagree"


def test_static_library_is_built_too():
    assert os.path.exists(os.path.join(ROOT, "frink_amd", "lib", "libfrink_hip.a"))


# crates/frink-core/src/weight_matrix/gpu_backend.rs:1265 -- has_launch == matvec_kernel.is_some(), every kind
def test_every_kind_the_backend_claims_can_be_launched():
    for kind in range(0, 40):
        name = fa.matvec_kernel(kind)
        assert bool(fa.lib().frk_hip_has_launch(kind)) == (name is not None)
        if kind in fa.KIND_NAME:
            assert name == fa.KIND_NAME[kind]
            assert (fa.lib().frk_hip_block_bytes(kind), fa.lib().frk_hip_block_elems(kind)) == fa.BLOCK[kind]
        else:
            assert name is None and fa.lib().frk_hip_block_bytes(kind) == 0
    assert all(fa.lib().frk_hip_gemm_supported(k) for k in (fa.Q4_0, fa.Q4_K, fa.Q5_K, fa.Q6_K, fa.Q8_0, fa.Q5_0, fa.MXFP4))
    assert fa.lib().frk_hip_gemm_supported(fa.IQ4_XS)
    assert not fa.lib().frk_hip_worth_a_gemm(1) and fa.lib().frk_hip_worth_a_gemm(2)


def test_an_unknown_kind_is_the_none_answer_not_an_error():
    assert fa.launch_matvec(3, np.zeros(20, np.uint8), np.zeros(32, np.float32), 1, 20) is None  # Q4_1


# crates/frink-core/src/weight_matrix/gpu_backend.rs:1342-1670: a mismatched shape is an error value, never a crash
@pytest.mark.parametrize("kind,rows,row_bytes,wlen,xlen,needle", [
    (fa.Q4_K, 0, 144, 0, 256, "rows=0"),
    (fa.Q4_K, 4, 143, 4 * 143, 256, "whole number"),
    (fa.Q4_K, 4, 144, 4 * 144 - 1, 256, "weights are"),
    (fa.Q4_K, 4, 144, 4 * 144, 255, "activation has"),
    (fa.Q6_K, 2, 420, 2 * 420, 256, "activation has"),
    (fa.Q8_0, 2, 35, 70, 32, "whole number"),
])
def test_shape_violations_are_refused_before_any_launch(kind, rows, row_bytes, wlen, xlen, needle):
    with pytest.raises(fa.BackendError) as e:
        fa.launch_matvec(kind, np.zeros(max(wlen, 1), np.uint8)[:wlen], np.zeros(xlen, np.float32), rows, row_bytes)
    assert e.value.code == fa.ERR_SHAPE and needle in e.value.message


def test_mul_mm_validate_shape():
    w = np.zeros(4 * 144, np.uint8)
    x = np.zeros(2 * 256, np.float32)
    for args, needle in [((0, 256, 2, 144), "empty shape"), ((4, 255, 2, 144), "not a multiple"),
                         ((4, 256, 2, 288), "row_bytes"), ((5, 256, 2, 144), "weights too small"),
                         ((4, 256, 3, 144), "activations too small")]:
        with pytest.raises(fa.BackendError) as e:
            fa.launch_mul_mm(fa.Q4_K, w, x, *args)
        assert e.value.code == fa.ERR_SHAPE and needle in e.value.message, e.value.message


def test_null_arguments_are_errors():
    L = fa.lib()
    assert L.frk_hip_probe(None) == fa.ERR_ARG
    assert L.frk_hip_gemv_dev(None, None, None, 0, None) == fa.ERR_ARG
    assert L.frk_hip_weights_release(None) == fa.OK
    assert L.frk_hip_weights_keep_decoded(None, None) == fa.ERR_ARG
    h = C.c_void_p()
    assert L.frk_hip_weights_register(fa.Q4_K, None, 144, 1, 256, C.byref(h)) == fa.ERR_ARG
    buf = np.zeros(144, np.uint8)
    assert L.frk_hip_weights_register(fa.Q4_K, C.c_void_p(buf.ctypes.data), 144, 1, 255, C.byref(h)) == fa.ERR_SHAPE
    assert L.frk_hip_weights_register(5, C.c_void_p(buf.ctypes.data), 144, 1, 256, C.byref(h)) == fa.ERR_UNSUPPORTED


def _have_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


@pytest.mark.skipif(_have_gpu(), reason="only meaningful on a GPU-less host")
def test_probe_on_a_gpu_less_host_is_an_error_value():
    with pytest.raises(fa.BackendError) as e:
        fa.probe()
    assert e.value.code == fa.ERR_NO_DEVICE
    # a well-formed launch then fails the same way instead of crashing
    w = np.zeros(144, np.uint8)
    with pytest.raises(fa.BackendError) as e:
        fa.launch_matvec(fa.Q4_K, w, np.zeros(256, np.float32), 1, 144)
    assert e.value.code == fa.ERR_NO_DEVICE


def test_forced_off_never_opens_a_device():
    # crates/frink-core/src/weight_matrix/gpu_backend.rs:1093-1104 -- run in a child so the
    # once-per-process decision is taken with the variable set
    import subprocess
    import sys
    code = ("import os,sys; sys.path.insert(0, %r); os.environ['FRINK_HIP']='off'; import frink_amd as fa; "
            "print(fa.lib().frk_hip_dense_enabled())" % ROOT)
    out = subprocess.check_output([sys.executable, "-c", code], text=True)
    assert out.strip() == "0"


def _host_check_binary():
    from frink_amd import build as fb
    if not os.path.exists(fb.HOST_CHECK_BIN):
        fb.build_host_check()
    return fb.HOST_CHECK_BIN


def test_cpp_host_mirror_without_a_device():
    """frink_amd/host/frink_hip.hpp (the C++ form of BackendCaps / BackendDispatch) driven by
    tests/host_mirror_check.cpp: capability tables agree over all 23 kinds, None vs Some(Err),
    shape errors before launch, FRINK_HIP=off."""
    import subprocess
    env = dict(os.environ, FRINK_HIP="off")
    r = subprocess.run([_host_check_binary()], env=env, text=True, capture_output=True, timeout=120)
    assert r.returncode == 0 and "FAIL" not in r.stdout, r.stdout + r.stderr
    assert "FRINK_HIP=off disables the backend" in r.stdout
