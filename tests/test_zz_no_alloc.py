"""ttmi_matmul_bfp_static: the GEMM entry point that allocates nothing (its scratch is a static device array), through the
C ABI, against ttmi_matmul_bfp on the same inputs — bit for bit, on two calls in a row, the second with a smaller input."""
import ctypes

import numpy as np
import pytest

torch = pytest.importorskip("torch")
from ttmi import capi, workloads  # noqa: E402

pytestmark = pytest.mark.gpu
BFP8, BFP4 = capi.BFLOAT8_B, capi.BFLOAT4_B
STATIC_BYTES = 16 << 20


def bf16_dev(bits_u16):
    return torch.from_numpy(np.ascontiguousarray(bits_u16.view(np.int16))).cuda().view(torch.bfloat16)


def both_entry_points(fmt, batch, b_batch, m, k, n, seed, bias=False, activation=capi.ACT_NONE, layout=capi.ROW_MAJOR):
    L = capi.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    a = bf16_dev(workloads.activations_bf16(m, k, seed=seed, batch=batch))
    if layout == capi.TILE:
        a = capi.tilize(a.reshape(batch, m, k))
    words = capi.pack_tensor(fmt, torch.from_numpy(workloads.weights_f32(k, n, seed=seed + 1, batch=b_batch)).cuda())
    bias_dev = bf16_dev(workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=seed + 2))) if bias else None
    bias_ptr = bias_dev.data_ptr() if bias else None
    outs = []
    for static in (False, True):
        c = torch.full((batch * m * n,), float("nan"), dtype=torch.bfloat16, device="cuda")
        common = (a.data_ptr(), layout, words.data_ptr(), fmt, batch, b_batch, m, k, n, bias_ptr, activation, c.data_ptr(), layout, capi.BFLOAT16)
        if static:
            capi.check(L.ttmi_matmul_bfp_static(*common, stream))
        else:
            capi.check(L.ttmi_matmul_bfp(*common, None, 0, stream))
        outs.append(c)
    torch.cuda.synchronize()
    capi.device_status()
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16)), (fmt, batch, m, k, n)


def test_static_scratch_matches_the_allocating_entry_point():
    # outputs shared between workgroups (partial-sum slots in the static array), first the larger input, then a smaller one
    both_entry_points(BFP8, 1, 1, 32, 4544, 4608, seed=200, layout=capi.TILE)
    both_entry_points(BFP8, 1, 1, 32, 1024, 288, seed=203)
    both_entry_points(BFP4, 2, 2, 24, 2048, 160, seed=206, bias=True, activation=capi.ACT_SILU)
    # several bands of rows (64-column kernel), then a single small band again
    both_entry_points(BFP8, 1, 1, 64, 4096, 512, seed=209)
    both_entry_points(BFP4, 1, 1, 8, 512, 64, seed=212)
    # no scratch at all (fused tiled kernels), and a shape whose expanded weights (2 bytes each) fit the array
    both_entry_points(BFP8, 1, 1, 256, 256, 256, seed=215, bias=True, activation=capi.ACT_GELU)
    both_entry_points(BFP8, 1, 1, 512, 128, 160, seed=218)
    both_entry_points(BFP8, 1, 1, 32, 2048, 320, seed=221)


def test_shapes_beyond_the_static_array_are_rejected_without_a_launch():
    L = capi.lib()
    need = L.ttmi_matmul_bfp_workspace_bytes(1, 2048, 4096, 14336, BFP8)
    assert need > STATIC_BYTES
    one = ctypes.c_void_p(256)
    assert L.ttmi_matmul_bfp_static(one, 0, one, BFP8, 1, 1, 2048, 4096, 14336, None, 0, one, 0, 0, None) == 3       # TTMI_ERR_UNSUPPORTED
    assert b"static array" in L.ttmi_last_error()
    assert L.ttmi_matmul_bfp_static(one, 0, one, BFP8, 1, 1, 32, 33, 64, None, 0, one, 0, 0, None) == 1             # the usual argument checks
    for shape in ((1, 32, 4544, 18176), (1, 32, 18176, 4544), (1, 32, 14336, 4096), (1, 64, 18176, 4544)):
        assert L.ttmi_matmul_bfp_workspace_bytes(*shape, BFP8) <= STATIC_BYTES, shape                               # the decode shapes fit
