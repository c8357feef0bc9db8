"""The C++ host layer (mllm-compatible Backend / op factories) seen through its C doorway.

CPU part: library loads, plugin descriptor is well-formed, failure paths behave like the reference's runtime
(unknown backend terminates the process, wrong option type throws std::bad_cast).
GPU part: a Linear created with Backend::createOp(kLinear, ...) -> load -> X2X -> reshape -> setup -> forward gives the
oracle's numbers for every weight scheme, through the in-tree factory and through the plugin package."""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

from mllm_amd import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_LIB = os.path.join(ROOT, "mllm_amd", "lib", "libmllm_hip_backend.so")


def _host():
    L = C.CDLL(HOST_LIB)
    L.opPackageDescriptor.restype = C.c_void_p
    return L


class _Desc(C.Structure):
    _pack_ = 4
    _fields_ = [("version", C.c_int32), ("name", C.c_char * 256), ("device_type", C.c_int32),
                ("op_factories_count", C.c_int32), ("op_factories_names", (C.c_char * 256) * 256),
                ("create", C.c_void_p * 256), ("free", C.c_void_p * 256)]


def test_host_library_loads_and_describes_its_ops():
    L = _host()
    d = _Desc.from_address(L.opPackageDescriptor())
    assert d.version == 1 and d.name == b"MllmHipQLinear"
    assert d.device_type == 4097 and d.op_factories_count == 2
    assert d.op_factories_names[0].value == b"hip_linear" and d.op_factories_names[1].value == b"hip_matmul"
    assert d.create[0] and d.free[0] and d.create[1] and d.free[1]
    assert C.sizeof(_Desc) == 4 + 256 + 4 + 4 + 256 * 256 + 2 * 256 * 8


def test_wrong_option_type_throws_bad_cast():
    assert _host().mllm_hip_backend_probe_bad_cast() == 1


def test_unknown_backend_terminates_process():
    code = "import ctypes; L = ctypes.CDLL(%r); L.mllm_hip_backend_probe_missing_backend()" % HOST_LIB
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert r.returncode == 1 and "Backend for device 4097 not found" in r.stderr


# ------------------------------------------------------------------------------------------------- GPU
def _run(L, scheme, W, scale, zp, bias, x, x_bf16, M, N, K, group, via_plugin):
    out_bf16 = scheme in ("w8a8", "w4a16")
    y = np.empty((M, N), np.uint16 if out_bf16 else np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p) if a is not None else None
    rc = L.mllm_hip_backend_run_linear(scheme.encode(), p(W), p(scale), p(zp), p(bias), p(x), int(x_bf16), p(y), M, N, K,
                                       group, 0, 1, int(via_plugin), HOST_LIB.encode())  # weights carry IEEE scale bits
    assert rc == (128 if out_bf16 else 0), rc  # returns the output dtype id: kBFloat16 = 128, kFloat32 = 0
    return y


@pytest.mark.gpu
@pytest.mark.parametrize("via_plugin", [0, 1])
def test_linear_through_the_op_factory(via_plugin):
    from oracle import oracle as orc
    from gpu_util import announce, rel_l2
    L = _host()
    rng = synth.rng_for(5, via_plugin)
    N, K = 192, 512
    for scheme, wtype in (("q4_0", 0), ("q8_0", 1)):
        W = synth.make_weight(rng, wtype, N, K)
        bias = rng.standard_normal(N).astype(np.float32)
        for M in (1, 5, 20):
            x = synth.make_x_fp32(rng, M, K)
            announce("host linear", scheme, M, "plugin", via_plugin)
            # up to 8 rows: the decode GEMV (fp32 block arithmetic); more: the matrix-core path (fp16 operands, about 2e-4)
            tol = 2e-6 if M <= 8 else 5e-4
            y = _run(L, scheme, W, None, None, bias, x, False, M, N, K, 0, via_plugin)
            assert rel_l2(y, orc.linear_q(x, W, wtype, bias, orc.SCALE_X86_REF)) < tol
            bits, xf = synth.make_x_bf16(rng, M, K)
            y = _run(L, scheme, W, None, None, None, bits, True, M, N, K, 0, via_plugin)
            assert rel_l2(y, orc.linear_q(xf, W, wtype, None, orc.SCALE_X86_REF)) < tol
    # W8A8
    M = 40
    a_bits, W8, ws = synth.make_w8a8(rng, M, N, K)
    announce("host linear w8a8")
    y = _run(L, "w8a8", W8, ws, None, None, a_bits, True, M, N, K, 0, via_plugin)
    q, s = orc.per_token_quant_int8(synth.bf16_bits_to_fp32(a_bits))
    assert np.array_equal(y, orc.w8a8_gemm(q, s, W8, ws)[1])
    # W4A16
    qw, sc, zp, _, _ = synth.make_w4a16(rng, N, K)
    bits, _ = synth.make_x_bf16(rng, M, K)
    biasb = synth.fp32_to_bf16_bits((rng.standard_normal(N) * 0.1).astype(np.float32))
    announce("host linear w4a16")
    y = _run(L, "w4a16", qw, sc, zp, biasb, bits, True, M, N, K, 128, via_plugin)
    want = orc.w4a16_gemm(bits, qw, sc, zp, biasb)
    assert rel_l2(synth.bf16_bits_to_fp32(y), synth.bf16_bits_to_fp32(want)) < 1e-3


@pytest.mark.gpu
def test_matmul_slot():
    from gpu_util import announce
    L = _host()
    rng = synth.rng_for(5, 9)
    M, N, K = 70, 130, 96
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal((N, K)).astype(np.float32)
    c = np.empty((M, N), np.float32)
    p = lambda t: t.ctypes.data_as(C.c_void_p)
    announce("host matmul")
    assert L.mllm_hip_backend_run_matmul(p(a), p(b), p(c), M, N, K, 1) == 0
    assert np.allclose(c, a @ b.T, rtol=1e-5, atol=1e-4)
    bt = np.ascontiguousarray(b.T)
    assert L.mllm_hip_backend_run_matmul(p(a), p(bt), p(c), M, N, K, 0) == 0
    assert np.allclose(c, a @ b.T, rtol=1e-5, atol=1e-4)
