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
        for M in (1, 5, 12, 20, 40, 60):
            x = synth.make_x_fp32(rng, M, K)
            announce("host linear", scheme, M, "plugin", via_plugin)
            # up to 48 rows: the decode GEMV, in groups of eight (fp32 block arithmetic); more: the matrix-core path (fp16
            # operands, about 2e-4)
            tol = 2e-6 if M <= 48 else 5e-4
            y = _run(L, scheme, W, None, None, bias, x, False, M, N, K, 0, via_plugin)
            assert rel_l2(y, orc.linear_q(x, W, wtype, bias, orc.SCALE_X86_REF)) < tol
            bits, xf = synth.make_x_bf16(rng, M, K)
            y = _run(L, scheme, W, None, None, None, bits, True, M, N, K, 0, via_plugin)
            assert rel_l2(y, orc.linear_q(xf, W, wtype, None, orc.SCALE_X86_REF)) < tol
    # K-quants
    for scheme, wtype in (("q4_k", 2), ("q6_k", 3)):
        W = synth.make_weight(rng, wtype, N, K)
        bias = rng.standard_normal(N).astype(np.float32)
        for M in (1, 5, 20):
            x = synth.make_x_fp32(rng, M, K)
            announce("host linear", scheme, M)
            y = _run(L, scheme, W, None, None, bias, x, False, M, N, K, 0, via_plugin)
            # up to 8 rows the GEMV (integer / fp32 arithmetic), more the matrix-core path (fp16 operands, about 3.5e-4)
            assert rel_l2(y, orc.linear_kq(x, W, wtype, bias, orc.SCALE_X86_REF)) < (2e-6 if M <= 8 else 1e-3)
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


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
def test_matmul_slot_batched_in_one_launch(dtype):
    """[batch][M][K] x [batch][K][N] (attention probabilities x values) and a transposed left operand through the kMatMul slot"""
    import torch
    from gpu_util import announce
    L = _host()
    rng = synth.rng_for(5, 10)
    batch, M, N, K = 6, 40, 64, 50
    td, tid = {"fp32": (torch.float32, 0), "bf16": (torch.bfloat16, 128), "fp16": (torch.float16, 1)}[dtype]
    a = torch.from_numpy(rng.standard_normal((batch, M, K)).astype(np.float32)).to(td)
    b = torch.from_numpy(rng.standard_normal((batch, K, N)).astype(np.float32)).to(td)
    c = torch.empty((batch, M, N), dtype=td)
    want = (a.double() @ b.double()).numpy()
    tol = {"fp32": 2e-6, "bf16": 3e-3, "fp16": 4e-4}[dtype]
    vp = lambda t: C.c_void_p(t.data_ptr())
    announce("host matmul batched " + dtype)
    assert L.mllm_hip_backend_run_matmul_batched(vp(a), vp(b), vp(c), tid, batch, M, N, K, 0, 0, 1) == 0
    assert np.linalg.norm(c.double().numpy() - want) / np.linalg.norm(want) <= tol
    at = a.transpose(1, 2).contiguous()
    c.zero_()
    assert L.mllm_hip_backend_run_matmul_batched(vp(at), vp(b), vp(c), tid, batch, M, N, K, 1, 0, 1) == 0
    assert np.linalg.norm(c.double().numpy() - want) / np.linalg.norm(want) <= tol


# ---- model files -------------------------------------------------------------------------------------------------------
# Writers restated from the file layouts (mllm/core/schema/ModelFileV1.hpp:36-52, ModelFileV2.hpp:40-62; struct formats as
# pymllm/mobile/convertor/model_file_v2.py:68-99 packs them).  dtype ids: mllm/core/DataTypes.hpp (kFloat32 0, kFloat16 1,
# kGGUF_Q4_0 2, kGGUF_Q8_0 8, kInt8 16, kBFloat16 128, kUInt8 129).
import struct

_DT = {"f32": 0, "f16": 1, "q4_0": 2, "q8_0": 8, "i8": 16, "bf16": 128, "u8": 129}


def _write_v1(path, tensors):
    """tensors: list of (name, dtype id, shape, bytes)"""
    desc = sum(4 + len(n.encode()) + 8 + 8 + 4 for n, _, _, _ in tensors)
    off = 12 + desc
    with open(path, "wb") as f:
        f.write(struct.pack("<iQ", 20012, desc))
        for n, dt, _, b in tensors:
            nb = n.encode()
            f.write(struct.pack("<I", len(nb)) + nb + struct.pack("<QQi", len(b), off, dt))
            off += len(b)
        for _, _, _, b in tensors:
            f.write(b)


def _write_v2(path, tensors, extra=b""):
    off = 532 + len(extra) + 352 * len(tensors)
    with open(path, "wb") as f:
        f.write(struct.pack("<II512sIQ", 0x519A, 2, b"test-model".ljust(512, b"\0"), len(tensors), 532 + len(extra)))
        f.write(extra)
        for i, (n, dt, shape, b) in enumerate(tensors):
            f.write(struct.pack("<IIQQQ16i256s", i, dt, len(b), off, len(shape), *(list(shape) + [0] * (16 - len(shape))),
                                n.encode().ljust(256, b"\0")))
            off += len(b)
        for _, _, _, b in tensors:
            f.write(b)


def _file_tensor(L, path, version, name):
    L.mllm_hip_host_file_tensor.restype = C.c_int64
    dt, rank = C.c_int32(), C.c_int32()
    shape = (C.c_int32 * 16)()
    n = L.mllm_hip_host_file_tensor(path.encode(), version, name.encode(), C.byref(dt), C.byref(rank), shape, None,
                                    C.c_uint64(0))
    if n < 0:
        return None
    buf = (C.c_uint8 * max(n, 1))()
    assert L.mllm_hip_host_file_tensor(path.encode(), version, name.encode(), C.byref(dt), C.byref(rank), shape, buf,
                                       C.c_uint64(n)) == n
    return dt.value, list(shape[:rank.value]), bytes(buf[:n])


def _linear_file_tensors(rng, wtype, N, K):
    W = synth.make_weight(rng, wtype, N, K)
    bias = rng.standard_normal(N).astype(np.float32)
    name = "model.layers.3.mlp.down_proj"
    return W, bias, name, [(name + ".weight", _DT["q4_0"] if wtype == 0 else _DT["q8_0"], [N, K], W.tobytes()),
                           (name + ".bias", _DT["f32"], [N], bias.tobytes()),
                           ("model.norm.weight", _DT["f16"], [K], rng.standard_normal(K).astype(np.float16).tobytes())]


def test_model_file_readers_and_writers(tmp_path):
    """V1 and V2 files written here are read back tensor for tensor (dtype, shape, bytes); a file converted by the library
    (V1 -> V2 -> V1) is parsed here and holds the same tensors; a V2 file with an extra data segment in front of the
    descriptors is read; a missing tensor reports so."""
    L = _host()
    rng = synth.rng_for(5, 31)
    W, bias, name, tensors = _linear_file_tensors(rng, 0, 48, 96)
    p1, p2, p2x = str(tmp_path / "m1.mllm"), str(tmp_path / "m2.mllm"), str(tmp_path / "m2x.mllm")
    _write_v1(p1, tensors)
    _write_v2(p2, tensors)
    _write_v2(p2x, tensors, extra=b"\xab" * 100)
    for n, dt, shape, b in tensors:
        got1 = _file_tensor(L, p1, 1, n)
        numel = int(np.prod(shape))
        assert got1 == (dt, [numel], b)                       # V1 carries no shapes: flat, element count from the byte length
        assert _file_tensor(L, p2, 2, n) == (dt, shape, b)
        assert _file_tensor(L, p2x, 2, n) == (dt, shape, b)
    assert _file_tensor(L, p2, 2, "no.such.tensor") is None
    # library-side conversion, parsed independently here
    c2, c1 = str(tmp_path / "c2.mllm"), str(tmp_path / "c1.mllm")
    # read with mmap (the reference's default) the tensors are views into the mapping, with the bytes a plain read gives
    for path, version in ((p1, 1), (p2, 2)):
        for tname, _, _, _ in tensors:
            assert L.mllm_hip_host_file_tensor_is_mapped_view(path.encode(), version, tname.encode()) == 1
        assert L.mllm_hip_host_file_tensor_is_mapped_view(path.encode(), version, b"no.such.tensor") == -1
    assert L.mllm_hip_host_file_convert(p1.encode(), 1, c2.encode(), 2) == 3
    assert L.mllm_hip_host_file_convert(c2.encode(), 2, c1.encode(), 1) == 3
    raw = open(c2, "rb").read()
    magic, ver, _, num, doff = struct.unpack_from("<II512sIQ", raw, 0)
    assert (magic, ver, num, doff) == (0x519A, 2, 3, 532)
    seen = {}
    for i in range(num):
        pid, dt, size, off, slen, *rest = struct.unpack_from("<IIQQQ16i256s", raw, doff + 352 * i)
        seen[rest[16].rstrip(b"\0").decode()] = (dt, raw[off:off + size])
    for n, dt, shape, b in tensors:
        assert seen[n] == (dt, b)
    raw1 = open(c1, "rb").read()
    magic1, desc_len = struct.unpack_from("<iQ", raw1, 0)
    assert magic1 == 20012
    pos, names = 12, []
    while pos < 12 + desc_len:
        (nl,) = struct.unpack_from("<I", raw1, pos)
        nm = raw1[pos + 4:pos + 4 + nl].decode()
        ln, off, dt = struct.unpack_from("<QQi", raw1, pos + 4 + nl)
        pos += 4 + nl + 20
        names.append(nm)
        want = {n: (d, b) for n, d, _, b in tensors}[nm]
        assert (dt, raw1[off:off + ln]) == want
    assert sorted(names) == sorted(n for n, _, _, _ in tensors)


def _load_in_child(path, version, name, mmap):
    """mllm::load ends the process on a bad file (as the reference's MLLM_ERROR_EXIT does): run it in a child"""
    fn = "mllm_hip_host_file_tensor_is_mapped_view" if mmap else "mllm_hip_host_file_tensor"
    if mmap:
        call = "L.%s(%r, %d, %r)" % (fn, path.encode(), version, name.encode())
    else:
        call = ("L.%s(%r, %d, %r, ctypes.byref(ctypes.c_int32()), ctypes.byref(ctypes.c_int32()), (ctypes.c_int32 * 16)(), None, 0)"
                % (fn, path.encode(), version, name.encode()))
    code = "import ctypes; L = ctypes.CDLL(%r); L.%s.restype = ctypes.c_int64; print('rc', %s)" % (HOST_LIB, fn, call)
    return subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)


@pytest.mark.parametrize("mmap", [True, False])
def test_model_file_with_bad_offsets_is_refused(tmp_path, mmap):
    """Offsets and lengths in a model file are untrusted: a truncated file, an offset + length that wraps around 2^64, a
    descriptor count or descriptor length beyond the file, and a shape whose byte count overflows all end in the load
    error, never in a read outside the file."""
    rng = synth.rng_for(5, 77)
    _, _, name, tensors = _linear_file_tensors(rng, 0, 48, 96)
    wname = name + ".weight"
    good1, good2 = str(tmp_path / "g1.mllm"), str(tmp_path / "g2.mllm")
    _write_v1(good1, tensors)
    _write_v2(good2, tensors)
    for path, version in ((good1, 1), (good2, 2)):
        r = _load_in_child(path, version, wname, mmap)
        assert r.returncode == 0 and "rc" in r.stdout, r.stderr
    raw1, raw2 = open(good1, "rb").read(), open(good2, "rb").read()
    cases = []
    # truncated in the tensor data
    cases.append(("v1 truncated", 1, raw1[:len(raw1) - 40]))
    cases.append(("v2 truncated", 2, raw2[:len(raw2) - 40]))
    # V1: descriptor length beyond the file / enormous
    cases.append(("v1 desc_bytes huge", 1, raw1[:4] + struct.pack("<Q", 2**63) + raw1[12:]))
    cases.append(("v1 desc_bytes wraps", 1, raw1[:4] + struct.pack("<Q", 2**64 - 8) + raw1[12:]))
    # V1: first tensor's offset such that offset + length wraps to a small number
    (nl,) = struct.unpack_from("<I", raw1, 12)
    off_pos = 12 + 4 + nl + 8
    (ln,) = struct.unpack_from("<Q", raw1, 12 + 4 + nl)
    cases.append(("v1 offset wraps", 1, raw1[:off_pos] + struct.pack("<Q", 2**64 - ln + 16) + raw1[off_pos + 8:]))
    # V2: descriptor table offset wraps / count too large
    cases.append(("v2 desc offset wraps", 2, raw2[:524] + struct.pack("<Q", 2**64 - 352) + raw2[532:]))
    cases.append(("v2 count huge", 2, raw2[:520] + struct.pack("<I", 2**32 - 1) + raw2[524:]))
    # V2: every tensor's data offset wraps; every tensor's shape overflows the byte count
    bad = bytearray(raw2)
    for i in range(3):
        struct.pack_into("<Q", bad, 532 + 352 * i + 16, 2**64 - 64)
    cases.append(("v2 offset wraps", 2, bytes(bad)))
    bad = bytearray(raw2)
    for i in range(3):
        struct.pack_into("<Q", bad, 532 + 352 * i + 24, 16)
        struct.pack_into("<16i", bad, 532 + 352 * i + 32, *([2**31 - 1] * 16))
    cases.append(("v2 shape overflows", 2, bytes(bad)))
    for what, version, data in cases:
        path = str(tmp_path / "bad.mllm")
        open(path, "wb").write(data)
        r = _load_in_child(path, version, wname, mmap)
        assert r.returncode > 0 and "rc" not in r.stdout, (what, r.returncode, r.stdout, r.stderr)  # the exit code of the load error, not a signal
        assert "truncated" in r.stderr or "assertion failed" in r.stderr, (what, r.stderr)


@pytest.mark.gpu
@pytest.mark.parametrize("version", [1, 2])
def test_linear_from_model_file(tmp_path, version):
    """mllm::load -> createOp(kLinear) -> load(params) -> forward on a file holding reference Q4_0 / Q8_0 blocks"""
    from oracle import oracle as orc
    from gpu_util import announce, rel_l2
    L = _host()
    rng = synth.rng_for(5, 40 + version)
    N, K, M = 96, 256, 3
    for wtype in (0, 1):
        W, bias, name, tensors = _linear_file_tensors(rng, wtype, N, K)
        path = str(tmp_path / ("lin%d_%d.mllm" % (version, wtype)))
        (_write_v1 if version == 1 else _write_v2)(path, tensors)
        x = synth.make_x_fp32(rng, M, K)
        y = np.empty((M, N), np.float32)
        announce("linear from file", version, wtype)
        rc = L.mllm_hip_backend_run_linear_file(path.encode(), version, name.encode(), K, N, 1, x.ctypes.data_as(C.c_void_p), 0,
                                                y.ctypes.data_as(C.c_void_p), M, 0, 1)
        assert rc == 0  # kFloat32
        assert rel_l2(y, orc.linear_q(x, W, wtype, bias, orc.SCALE_X86_REF)) < 2e-6


@pytest.mark.gpu
@pytest.mark.parametrize("is_q8", [0, 1])
def test_decoder_mlp_through_the_op_factories(is_q8):
    """RMSNorm -> gate/up Linear -> SiLU -> Mul -> down Linear -> Add created through Backend::createOp: the oracle's chain
    within tolerance; with the image hand-over on, three Linear inputs arrive as quantized images and the result is the
    same bit for bit; softmax and top-k slots checked on the side"""
    from oracle import oracle as orc
    from gpu_util import announce, rel_l2
    L = _host()
    rng = synth.rng_for(5, 60 + is_q8)
    H, I, k = 256, 512, 4
    Wg, Wu, Wd = (synth.make_weight(rng, is_q8, I, H), synth.make_weight(rng, is_q8, I, H), synth.make_weight(rng, is_q8, H, I))
    nw = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    vp = lambda a: a.ctypes.data_as(C.c_void_p)
    for M in (1, 4, 8, 12, 24, 40, 60):
        x = synth.make_x_fp32(rng, M, H)
        ys, handed = [], []
        sm = np.empty((M, I), np.float32)
        ti = np.empty((M, k), np.int32)
        for fold in (0, 1):
            y = np.empty((M, H), np.float32)
            announce("decoder mlp", is_q8, M, "fold", fold)
            rc = L.mllm_hip_backend_run_decoder_mlp(is_q8, vp(Wg), vp(Wu), vp(Wd), vp(nw), vp(x), 0, vp(y), M, H, I, C.c_float(1e-6), fold,
                                                    vp(sm), vp(ti), k)
            assert rc >= 0, rc
            ys.append(y)
            handed.append(rc)
        assert handed == [0, 3 if M <= 8 else 0]
        assert np.array_equal(ys[0], ys[1])
        h = orc.rmsnorm(x, nw, 1e-6)
        g = orc.linear_q(h, Wg, is_q8, None, orc.SCALE_X86_REF)
        a = orc.silu(g) * orc.linear_q(h, Wu, is_q8, None, orc.SCALE_X86_REF)
        want = orc.linear_q(a, Wd, is_q8, None, orc.SCALE_X86_REF) + x
        # up to 48 rows every Linear is the fp32 block arithmetic.  More rows: the matrix-core Linear (fp16 operands, 2e-4 per
        # Linear on identical inputs, its own test); in a CHAIN the Q8_0 re-quantization in front of down_proj turns a
        # perturbation eps of its input into about sqrt(eps * 0.026) (codes flip at rounding boundaries), so the chain
        # is compared at 5e-3 and MLLM_HIP_PREFILL=blockdot keeps the fp32 arithmetic where that matters
        assert rel_l2(ys[0], want) < (1e-3 if M <= 48 else 5e-3)
        assert rel_l2(sm, orc.softmax(g)) < 1e-3
        assert np.array_equal(ti, orc.topk(sm, k, True, False)[1])


@pytest.mark.gpu
@pytest.mark.parametrize("external", [0, 1])
def test_linear_requantizes_after_a_write_the_backend_cannot_see(external):
    """RMSNorm -> Linear, then the activation tensor is overwritten by a plain hipMemcpy and the Linear runs again: the
    second result must follow the new contents.  With the backend's defaults no quantized image is kept at all (the
    hand-over is opt-in); with the hand-over on, a caller-owned buffer (external) never gets one either."""
    from oracle import oracle as orc
    from gpu_util import announce, rel_l2
    L = _host()
    rng = synth.rng_for(5, 90 + external)
    M, H, N = 4, 256, 320
    W = synth.make_weight(rng, 0, N, H)
    nw = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    x = synth.make_x_fp32(rng, M, H)
    h2 = synth.make_x_fp32(rng, M, H) * 3
    y1, y2 = np.empty((M, N), np.float32), np.empty((M, N), np.float32)
    vp = lambda a: a.ctypes.data_as(C.c_void_p)
    announce("rewrite behind the backend", external)
    rc = L.mllm_hip_backend_run_rewrite_behind_backend(0, vp(W), vp(nw), vp(x), vp(h2), vp(y1), vp(y2), M, H, N, external)
    assert rc == 0, rc  # no image for the tensor at the second call
    assert rel_l2(y1, orc.linear_q(orc.rmsnorm(x, nw, 1e-6), W, 0, None, orc.SCALE_X86_REF)) < 2e-6
    assert rel_l2(y2, orc.linear_q(h2, W, 0, None, orc.SCALE_X86_REF)) < 2e-6
