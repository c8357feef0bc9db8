"""GPU parity of the MatMul slot (activation x activation, mllm/backends/cpu/ops/MatMulOp.cpp:19-90).

fp32: exact products summed in fp32 on the matrix cores, against a float64 sum of the same products; the bound is a few
ulp of fp32 per sqrt(K) (rel-L2 <= 2e-6 written below).  bf16 / fp16: exact products, fp32 sums, one rounding; compared with
the float64 result rounded the same way (rel-L2 <= 1e-3, the bound the quantized Linears use)."""
import numpy as np
import pytest
import torch

from mllm_amd import qlinear as ql, synth
from gpu_util import announce, rel_l2

pytestmark = pytest.mark.gpu


def _ref(a, b, ta, tb):
    a64 = a.astype(np.float64)
    b64 = b.astype(np.float64)
    if ta:
        a64 = np.swapaxes(a64, -1, -2)
    if tb:
        b64 = np.swapaxes(b64, -1, -2)
    return a64 @ b64


SHAPES = [(1, 1, 1, 1), (1, 70, 130, 96), (3, 33, 65, 31), (2, 128, 128, 128), (5, 1, 257, 64), (2, 200, 7, 40),
          (4, 129, 131, 250), (1, 64, 64, 2049),
          # up to four rows against [K][N] (a decode token's probabilities x values): the GEMV form when not transposed
          (32, 1, 128, 1024), (3, 2, 136, 300), (2, 4, 1024, 257), (1, 3, 2052, 512), (5, 1, 8, 4096)]


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("batch,M,N,K", SHAPES)
def test_matmul_fp32(batch, M, N, K, ta, tb):
    rng = synth.rng_for(6, batch + M + N + K + 2 * ta + tb)
    a = rng.standard_normal((batch, K, M) if ta else (batch, M, K)).astype(np.float32)
    b = rng.standard_normal((batch, N, K) if tb else (batch, K, N)).astype(np.float32)
    announce("matmul fp32 %s ta=%d tb=%d" % ((batch, M, N, K), ta, tb))
    c = ql.matmul(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), ta, tb).cpu().numpy()
    assert c.shape == (batch, M, N)
    assert rel_l2(c, _ref(a, b, ta, tb)) <= 2e-6


def test_matmul_fp32_integers_are_exact_and_batches_do_not_mix():
    """small integers: every product and partial sum is exact in fp32, so the result must equal the integer product; each
    batch entry carries a different multiplier so that a wrong stride shows"""
    rng = synth.rng_for(6, 1)
    batch, M, N, K = 6, 96, 160, 72
    a = rng.integers(-8, 9, (batch, M, K)).astype(np.float32) * (1 + np.arange(batch, dtype=np.float32))[:, None, None]
    b = rng.integers(-8, 9, (batch, N, K)).astype(np.float32)
    announce("matmul fp32 exact")
    c = ql.matmul(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), False, True).cpu().numpy()
    assert np.array_equal(c, _ref(a, b, False, True).astype(np.float32))
    # one right-hand matrix for the whole batch
    c1 = ql.matmul(torch.from_numpy(a).cuda(), torch.from_numpy(b[2]).cuda(), False, True).cpu().numpy()
    assert np.array_equal(c1, _ref(a, b[2][None], False, True).astype(np.float32))


def test_matmul_unaligned_views_take_the_element_path():
    """operands that start 4 bytes into an allocation, and odd leading dimensions"""
    rng = synth.rng_for(6, 2)
    M, N, K = 50, 40, 37
    a = rng.standard_normal(M * K + 1).astype(np.float32)
    b = rng.standard_normal(N * K + 1).astype(np.float32)
    ad, bd = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    announce("matmul fp32 unaligned")
    c = ql.matmul(ad[1:].view(M, K), bd[1:].view(N, K), False, True).cpu().numpy()
    assert rel_l2(c, _ref(a[1:].reshape(M, K), b[1:].reshape(N, K), False, True)) <= 2e-6


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("batch,M,N,K", [(1, 70, 130, 96), (3, 33, 65, 31), (2, 256, 128, 128), (16, 128, 256, 64), (2, 9, 200, 1000),
                                          (32, 1, 128, 1024), (3, 2, 136, 300), (2, 4, 1024, 264), (1, 3, 4104, 512)])
def test_matmul_16_bit(batch, M, N, K, ta, tb, dtype):
    rng = synth.rng_for(6, 1000 + batch + M + N + K + 2 * ta + tb)
    td = torch.bfloat16 if dtype == "bf16" else torch.float16
    a = torch.from_numpy(rng.standard_normal((batch, K, M) if ta else (batch, M, K)).astype(np.float32)).to(td)
    b = torch.from_numpy(rng.standard_normal((batch, N, K) if tb else (batch, K, N)).astype(np.float32)).to(td)
    announce("matmul %s %s ta=%d tb=%d" % (dtype, (batch, M, N, K), ta, tb))
    c = ql.matmul(a.cuda(), b.cuda(), ta, tb).cpu()
    want = torch.from_numpy(_ref(a.float().numpy(), b.float().numpy(), ta, tb)).to(td)
    assert rel_l2(c.float().numpy(), want.float().numpy()) <= 1e-3
    # and against the unrounded float64 result: no worse than one rounding of the result type
    assert rel_l2(c.float().numpy(), _ref(a.float().numpy(), b.float().numpy(), ta, tb)) <= (3e-3 if dtype == "bf16" else 4e-4)
