"""The entry point that allocates nothing (mllm_hip_linear_q_gemv_multi_static): its workspace (the quantized-activation
image and, where they fit, the partial sums of the K slices) is a static device array of the library instead of a
caller-provided buffer.  Called through the C ABI and compared bit for bit with the entry point it is a variant of
(mllm_hip_linear_q_gemv_multi_wsn with a workspace of the array's size), on two calls in a row, the second with a smaller
input, which must not see anything the first one left in the array."""
import ctypes as C

import numpy as np
import pytest
import torch

from mllm_amd import _lib, qlinear as ql, synth
from gpu_util import announce, bf16_dev, to_dev

pytestmark = pytest.mark.gpu

STATIC_BYTES = 327680  # the library's static array (include/mllm_hip_qlinear.h)


def _both(wtype, Ws, bits_or_x, M, K, is_bf16):
    """runs the static entry point and the workspace one on the same inputs; returns (static outputs, workspace outputs)."""
    L = _lib.lib()
    ws = [ql.PackedQWeight(wtype, torch.from_numpy(W)) for W in Ws]
    x = bf16_dev(bits_or_x) if is_bf16 else to_dev(bits_or_x)
    outs = []
    for static in (True, False):
        ys = [torch.full((M, w.N), float("nan"), dtype=torch.float32, device="cuda") for w in ws]
        parts = (_lib.GemvPart * len(ws))()
        for i, w in enumerate(ws):
            parts[i] = _lib.GemvPart(w.ptr, None, ys[i].data_ptr(), w.N)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        if static:
            rc = L.mllm_hip_linear_q_gemv_multi_static(wtype, len(ws), parts, x.data_ptr(), 1 if is_bf16 else 0, M, K,
                                                       ql.SCALE_X86_REF, stream)
        else:
            work = torch.empty(STATIC_BYTES, dtype=torch.uint8, device="cuda")  # the size of the library's static array
            rc = L.mllm_hip_linear_q_gemv_multi_wsn(wtype, len(ws), parts, x.data_ptr(), 1 if is_bf16 else 0, M, K,
                                                    ql.SCALE_X86_REF, work.data_ptr(), STATIC_BYTES, stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        outs.append([y.cpu().numpy() for y in ys])
    return outs


@pytest.mark.parametrize("wtype", [0, 1])
def test_static_scratch_gemv_equals_workspace_gemv_on_two_calls_in_a_row(wtype):
    _lib.check(_lib.lib().mllm_hip_init(0), "mllm_hip_init")
    rng = synth.rng_for(7, 40 + wtype)
    # first call: eight bf16 rows of a long K through two sibling matrices (uses the whole image of eight rows)
    M, K = 8, 9728
    Ws = [synth.make_weight(rng, wtype, 2560, K), synth.make_weight(rng, wtype, 96, K)]
    bits, _ = synth.make_x_bf16(rng, M, K)
    announce("static gemv, first call", wtype, M, K)
    got, want = _both(wtype, Ws, bits, M, K, True)
    for g, w in zip(got, want):
        assert not np.isnan(g).any()
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32))
    # second call: fewer, shorter fp32 rows; whatever the first call left in the array must not matter
    M, K = 5, 2560
    Ws = [synth.make_weight(rng, wtype, 1024, K)]
    x = synth.make_x_fp32(rng, M, K)
    announce("static gemv, second call", wtype, M, K)
    got, want = _both(wtype, Ws, x, M, K, False)
    assert np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32))
    # and a many-row call: passes of eight rows over the same array, in stream order
    M, K = 19, 2560
    x = synth.make_x_fp32(rng, M, K)
    announce("static gemv, 19 rows", wtype, M, K)
    got, want = _both(wtype, Ws, x, M, K, False)
    assert np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32))
