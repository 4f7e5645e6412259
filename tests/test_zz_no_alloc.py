"""ttmi_matmul_bfp_static: the GEMM entry point that allocates nothing (its scratch is a static device array), through the
C ABI, against ttmi_matmul_bfp on the same inputs — bit for bit, on two calls in a row, the second with a smaller input — and
that it allocates nothing: on a stream the library has never seen (where the allocating entry point would allocate) the
library's count of its own allocations stays put, and the device's free memory does not move across a call."""
import ctypes
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

torch = pytest.importorskip("torch")
from ttmi import capi, workloads  # noqa: E402

pytestmark = pytest.mark.gpu
BFP8, BFP4 = capi.BFLOAT8_B, capi.BFLOAT4_B
STATIC_BYTES = 16 << 20


def bf16_dev(bits_u16):
    return torch.from_numpy(np.ascontiguousarray(bits_u16.view(np.int16))).cuda().view(torch.bfloat16)


def both_entry_points(fmt, batch, b_batch, m, k, n, seed, bias=False, activation=capi.ACT_NONE, layout=capi.ROW_MAJOR, out_bfp=None):
    L = capi.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    a = bf16_dev(workloads.activations_bf16(m, k, seed=seed, batch=batch))
    if layout == capi.TILE:
        a = capi.tilize(a.reshape(batch, m, k))
    words = capi.pack_tensor(fmt, torch.from_numpy(workloads.weights_f32(k, n, seed=seed + 1, batch=b_batch)).cuda())
    bias_dev = bf16_dev(workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=seed + 2))) if bias else None
    bias_ptr = bias_dev.data_ptr() if bias else None
    outs = []
    out_dtype, out_bytes = (capi.BFLOAT16, batch * m * n * 2) if out_bfp is None else (out_bfp, batch * (m // 32) * (n // 32) * (1088 if out_bfp == BFP8 else 576))
    for static in (False, True):
        c = torch.full((out_bytes,), 0xFF, dtype=torch.uint8, device="cuda")
        common = (a.data_ptr(), layout, words.data_ptr(), fmt, batch, b_batch, m, k, n, bias_ptr, activation, c.data_ptr(), layout, out_dtype)
        if static:
            # On a stream that the library has never seen, where the allocating entry point would have to allocate: the
            # device's free memory must not move across the call (the first static call on a device resolves the array's
            # address, nothing more).
            fresh = torch.cuda.Stream()
            fresh.wait_stream(torch.cuda.current_stream())
            torch.cuda.synchronize()
            L.ttmi_test_allocations.restype = ctypes.c_uint64
            made_before = L.ttmi_test_allocations()
            capi.check(L.ttmi_matmul_bfp_static(*common, ctypes.c_void_p(fresh.cuda_stream)))
            # Whatever device memory the first launch on a new stream costs is the runtime's (the stream's queue, scratch for
            # a kernel that spills registers); a second call on it must not move the device's free memory by a byte.
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            capi.check(L.ttmi_matmul_bfp_static(*common, ctypes.c_void_p(fresh.cuda_stream)))
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before, "device memory moved across ttmi_matmul_bfp_static"
            assert L.ttmi_test_allocations() == made_before, "ttmi_matmul_bfp_static made the library allocate"
        else:
            capi.check(L.ttmi_matmul_bfp(*common, None, 0, stream))
        outs.append(c)
    torch.cuda.synchronize()
    capi.device_status()
    if out_bfp is None:
        assert not torch.isnan(outs[0].view(torch.bfloat16).float()).any()
    assert torch.equal(outs[0], outs[1]), (fmt, batch, m, k, n)


def test_static_scratch_matches_the_allocating_entry_point(test_library):        # the test build: it counts the library's allocations
    # outputs shared between workgroups (partial-sum slots in the static array), first the larger input, then a smaller one
    both_entry_points(BFP8, 1, 1, 32, 4544, 4608, seed=200, layout=capi.TILE)
    both_entry_points(BFP8, 1, 1, 32, 1024, 288, seed=203)
    both_entry_points(BFP4, 2, 2, 24, 2048, 160, seed=206, bias=True, activation=capi.ACT_SILU)
    # two bands of rows per workgroup (two slots each), three bands (64-column kernel), then a single small band again
    both_entry_points(BFP8, 1, 1, 64, 4096, 512, seed=209)
    both_entry_points(BFP8, 1, 1, 96, 1024, 2048, seed=210)
    both_entry_points(BFP4, 1, 1, 8, 512, 64, seed=212)
    # no scratch at all (fused tiled kernels), a shape whose expanded weights (2 bytes each) fit the array — they overwrite
    # the slots, which the next launch that shares outputs has to find empty again
    both_entry_points(BFP8, 12, 12, 384, 256, 256, seed=215, bias=True, activation=capi.ACT_GELU)
    both_entry_points(BFP8, 1, 1, 1024, 128, 4096, seed=218)
    both_entry_points(BFP8, 1, 1, 32, 2048, 320, seed=221)
    # block-float outputs, whatever kernel the shape goes to: packed in the epilogue, no buffer in between
    both_entry_points(BFP8, 1, 1, 32, 2048, 320, seed=224, layout=capi.TILE, out_bfp=BFP8)
    both_entry_points(BFP8, 12, 12, 384, 256, 256, seed=227, layout=capi.TILE, out_bfp=BFP4)
    both_entry_points(BFP4, 1, 1, 1024, 128, 4096, seed=230, layout=capi.TILE, out_bfp=BFP8)
    both_entry_points(BFP8, 1, 1, 96, 4096, 512, seed=233, layout=capi.TILE, out_bfp=BFP8)


def test_static_entry_point_alone_in_a_fresh_process(oracle):
    """A process that calls nothing but ttmi_matmul_bfp_static — no allocating call, no ttmi_device_status before it, so the
    device has no error word and the array has never been filled — against the CPU oracle's weights."""
    import subprocess
    import sys

    program = r'''
import ctypes, sys
sys.path[:0] = [%r, %r]
import numpy as np, torch
from ttmi import capi, workloads
L = capi.lib()
m, k, n = 32, 2048, 320
a_bits = workloads.activations_bf16(m, k, seed=300)
w = workloads.weights_f32(k, n, seed=301)
a = torch.from_numpy(np.ascontiguousarray(a_bits.view(np.int16))).cuda().view(torch.bfloat16)
packed = np.load(sys.argv[1])
words = torch.from_numpy(packed).cuda()
c = torch.full((m * n,), float("nan"), dtype=torch.bfloat16, device="cuda")
for rep in range(2):
    rc = L.ttmi_matmul_bfp_static(a.data_ptr(), capi.ROW_MAJOR, words.data_ptr(), capi.BFLOAT8_B, 1, 1, m, k, n, None, 0, c.data_ptr(), capi.ROW_MAJOR, capi.BFLOAT16,
                                  ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, L.ttmi_last_error()
    torch.cuda.synchronize()
np.save(sys.argv[2], c.float().cpu().numpy())
''' % (ROOT, ROOT + "/tt-metal_amd")
    import os
    import tempfile

    m, k, n = 32, 2048, 320
    w = workloads.weights_f32(k, n, seed=301)
    packed = oracle.from_torch_bfp_tiles(BFP8, w)
    w_unpacked = oracle.to_torch_bfp_tiles(BFP8, packed, (k, n))
    with tempfile.TemporaryDirectory() as tmp:
        np.save(os.path.join(tmp, "w.npy"), packed.view(np.int32))
        done = subprocess.run([sys.executable, "-c", program, os.path.join(tmp, "w.npy"), os.path.join(tmp, "c.npy")], capture_output=True, text=True, timeout=300)
        assert done.returncode == 0, done.stderr[-2000:]
        c = np.load(os.path.join(tmp, "c.npy")).reshape(m, n)
    a = workloads.bf16_bits_to_f32(workloads.activations_bf16(m, k, seed=300)).astype(np.float64)
    ref = a @ w_unpacked.astype(np.float64)
    bound = 2.0 ** -8 * np.abs(ref) + 2.0 * k * 2.0 ** -24 * (np.abs(a) @ (5.0 * np.abs(w_unpacked).astype(np.float64).reshape(k, n // 16, 16).max(axis=2, keepdims=True).repeat(16, axis=2).reshape(k, n))) + 1e-30
    assert np.all(np.isfinite(c)) and np.all(np.abs(c - ref) <= bound)


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
