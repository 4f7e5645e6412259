"""GPU parity of the block-float-weight GEMM against an fp32/fp64 CPU matmul on oracle-unpacked weights.

Tolerance (stated by the task): PCC >= 0.9999 and, per element,
    |c - ref| <= 2**-8 * |ref| + 2 * K * 2**-24 * sum_k |a_k| |w_k|
(one bf16 rounding of the output, doubled, plus the classical fp32 summation bound).  The streaming kernels add and
subtract the face row's power of two with every weight, so for them the summation bound is over |w_k| + 4 x the largest
|w| of the 16-column face row (check_against_reference(face_row_scale=True), test_face_rows_with_outliers); with weights
whose face rows hold comparable magnitudes, as everywhere else in this file, they meet the bound above as well.
"""
import ctypes

import numpy as np
import pytest

torch = pytest.importorskip("torch")
from ttmi import capi, workloads  # noqa: E402

pytestmark = pytest.mark.gpu
BFP8, BFP4 = capi.BFLOAT8_B, capi.BFLOAT4_B
FMT = {"bfp8_b": BFP8, "bfp4_b": BFP4}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def bf16_dev(bits_u16):
    return dev(bits_u16.view(np.int16)).view(torch.bfloat16)


def comp_pcc(golden, calculated):
    """models/utility_functions.py:544-597 comp_pcc, for finite inputs."""
    g = golden.astype(np.float64).reshape(-1)
    c = calculated.astype(np.float64).reshape(-1)
    if np.array_equal(g, c):
        return 1.0
    return float(np.corrcoef(g, c)[0, 1])


def check_against_reference(c_f32, a_f32, w_f32, k, bf16_out=True, rows=None, face_row_scale=False):
    """|c - ref| <= output rounding (2^-8 |ref| for bf16, 2^-22 |ref| for fp32) + the worst case of 2K fp32 additions,
    2K 2^-24 (|A| . T), where T bounds the terms that are added: T = |W| for kernels that multiply by the expanded weights.
    The streaming kernels (face_row_scale) add A.hi and -A.lo with |2 hi| <= |W| + S, |2 lo| = S, S = 2^(E-126) <= 2 x the
    largest |W| of the 16-column face row: T = |W| + 4 x that maximum.  PCC >= 0.9999 either way."""
    a64, w64 = a_f32.astype(np.float64), w_f32.astype(np.float64)
    ref = np.matmul(a64, w64)
    terms = np.abs(w64)
    if face_row_scale:
        kk, nn = w64.shape[-2:]
        row_max = terms.reshape(-1, kk, nn // 16, 16).max(axis=3, keepdims=True).repeat(16, axis=3).reshape(w64.shape)
        terms = terms + 4.0 * row_max
    mag = np.matmul(np.abs(a64), terms)
    bound = (2.0 ** -8 if bf16_out else 2.0 ** -22) * np.abs(ref) + 2.0 * k * 2.0 ** -24 * mag + 1e-37
    got = c_f32.astype(np.float64)
    worst = float(np.max(np.abs(got - ref) / bound))
    assert worst <= 1.0, f"elementwise bound exceeded by factor {worst}"
    pcc = comp_pcc(ref, got)
    assert pcc >= 0.9999, pcc
    return pcc


def pack_weights(oracle, w_f32, fmt):
    """[..., K, N] fp32 -> (device packed words by the GPU packer, oracle-unpacked fp32 [..., K, N])."""
    words = capi.pack_tensor(fmt, dev(w_f32))
    want = oracle.from_torch_bfp_tiles(fmt, w_f32)
    assert np.array_equal(words.cpu().numpy().view(np.uint32), want)
    return words, oracle.to_torch_bfp_tiles(fmt, want, w_f32.shape)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("m,k,n", [(32, 32, 32), (32, 64, 128), (32, 160, 96), (7, 96, 160), (64, 256, 288), (45, 512, 64)])
def test_small_shapes_row_major(oracle, fmt, m, k, n):
    a_bits = workloads.activations_bf16(m, k, seed=60)
    w = workloads.weights_f32(k, n, seed=61)
    words, w_unpacked = pack_weights(oracle, w, fmt)
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n)
    torch.cuda.synchronize()
    check_against_reference(c.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)
    c32 = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n, out_dtype=torch.float32)
    check_against_reference(c32.cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k, bf16_out=False)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_identity_weights_return_the_activations(oracle, fmt):
    """tests/tt_metal/tt_metal/unit_tests/.../test_matmul_single_tile_bfp8b.cpp:121-129,168: x @ I == x, exactly."""
    m, k = 64, 96
    a_bits = workloads.activations_bf16(m, k, seed=62)
    words, w_unpacked = pack_weights(oracle, np.eye(k, dtype=np.float32), fmt)
    assert np.array_equal(w_unpacked, np.eye(k, dtype=np.float32))
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, fmt, 1, 1, m, k, k)
    assert np.array_equal(c.view(torch.int16).cpu().numpy().view(np.uint16)[0], a_bits)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_integer_valued_problem_is_exact(oracle, fmt):
    """Small integers: every product and partial sum is exact in fp32, so any summation order gives the same bits."""
    rng = np.random.default_rng(63)
    m, k, n = 32, 288, 160
    lim = 64 if fmt == BFP8 else 4
    a = rng.integers(-8, 9, size=(m, k)).astype(np.float32)
    w = rng.integers(-lim + 1, lim, size=(k, n)).astype(np.float32)
    w[:, ::16] = lim - 1 if fmt == BFP4 else 64.0      # every face row shares one exponent, so all values are kept exactly
    words, w_unpacked = pack_weights(oracle, w, fmt)
    assert np.array_equal(w_unpacked, w)
    c = capi.matmul_bfp(bf16_dev(workloads.f32_to_bf16_bits_rne(a)), capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n, out_dtype=torch.float32)
    assert np.array_equal(c.cpu().numpy()[0], a @ w)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_tile_layout_in_and_out(oracle, fmt):
    m, k, n = 64, 128, 192
    a_bits = workloads.activations_bf16(m, k, seed=64)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=65), fmt)
    a_tiles = capi.tilize(bf16_dev(a_bits))
    c_tiles = capi.matmul_bfp(a_tiles, capi.TILE, words, fmt, 1, 1, m, k, n, c_layout=capi.TILE)
    c_rm = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n)
    assert torch.equal(capi.untilize(c_tiles, (1, m, n)).view(torch.int16), c_rm.view(torch.int16))
    check_against_reference(c_rm.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)


@pytest.mark.parametrize("b_batch", [1, 3])
def test_batched_and_broadcast_weights(oracle, b_batch):
    batch, m, k, n = 3, 40, 96, 64
    a_bits = workloads.activations_bf16(m, k, seed=66, batch=batch)
    w = workloads.weights_f32(k, n, seed=67, batch=b_batch)
    words, w_unpacked = pack_weights(oracle, w, BFP8)
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP8, batch, b_batch, m, k, n)
    a = workloads.bf16_bits_to_f32(a_bits)
    for b in range(batch):
        check_against_reference(c[b].float().cpu().numpy(), a[b], w_unpacked[b if b_batch > 1 else 0], k)


@pytest.mark.parametrize("activation", [capi.ACT_NONE, capi.ACT_RELU, capi.ACT_GELU, capi.ACT_SILU])
def test_linear_bias_and_activation(oracle, activation):
    """ttnn.linear golden (ttnn/ttnn/operations/matmul.py:419-438): a @ w + bias, then the activation."""
    m, k, n = 32, 256, 128
    a_bits = workloads.activations_bf16(m, k, seed=68)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=69), BFP8)
    bias_bits = workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=70))
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n, bias=bf16_dev(bias_bits),
                        activation=activation, out_dtype=torch.float32)
    x = torch.from_numpy(workloads.bf16_bits_to_f32(a_bits).astype(np.float64) @ w_unpacked.astype(np.float64)
                         + workloads.bf16_bits_to_f32(bias_bits).astype(np.float64))
    ref = {capi.ACT_NONE: lambda t: t, capi.ACT_RELU: torch.relu, capi.ACT_GELU: torch.nn.functional.gelu,
           capi.ACT_SILU: torch.nn.functional.silu}[activation](x)
    assert torch.allclose(c[0].cpu().double(), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("m", [40, 24])      # two bands (64-column streaming kernel), one band (128-column kernel)
@pytest.mark.parametrize("workgroups", ["1", "3", "7", "64", "512", "4096"])
def test_any_number_of_workgroups_gives_the_same_bits(oracle, workgroups, m, knobs):
    """The k range of an output may be shared between workgroups in any way; partial sums are added in a fixed order."""
    k, n = 1024, 288
    a_bits = workloads.activations_bf16(m, k, seed=71)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=72), BFP8)
    knobs("workgroups", workgroups)
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)
    again = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)
    assert torch.equal(c.view(torch.int16), again.view(torch.int16))
    check_against_reference(c.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)


@pytest.mark.parametrize("m,k,n,fmt", [(32, 4544, 18176, BFP8), (32, 4096, 6144, BFP8), (64, 2048, 1024, BFP4), (24, 1024, 288, BFP8)])
def test_shared_outputs_inside_one_xcd_or_anywhere_give_the_same_bits(oracle, m, k, n, fmt, knobs):
    """Where consecutive workgroups are known to go to consecutive XCDs, the 128-column kernel places the workgroups that
    share an output in one XCD and hands partial sums over through that XCD's L2 (plain stores); otherwise through
    device-scope stores.  The sums are added in the same order either way: the same bits."""
    a_bits = workloads.activations_bf16(m, k, seed=75)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=76), fmt)
    a = bf16_dev(a_bits)
    knobs("kernel", "wide")
    placed = [capi.matmul_bfp(a, capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n).clone() for _ in range(3)]
    knobs("xcds", 1)
    anywhere = capi.matmul_bfp(a, capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n).clone()
    knobs("xcds", 8)
    placed.append(capi.matmul_bfp(a, capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n).clone())
    torch.cuda.synchronize()
    capi.device_status()
    for c in placed:
        assert torch.equal(c.view(torch.int16), anywhere.view(torch.int16))
    check_against_reference(anywhere.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)


def test_caller_workspace(oracle):
    m, k, n = 32, 2048, 256
    a_bits = workloads.activations_bf16(m, k, seed=73)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=74), BFP4)
    need = capi.lib().ttmi_matmul_bfp_workspace_bytes(1, m, k, n, BFP4)
    assert need > 0
    ws = torch.full((need,), 0x5A, dtype=torch.uint8, device="cuda")   # dirty on purpose
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP4, 1, 1, m, k, n, workspace=ws)
    check_against_reference(c.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)
    small = torch.empty(need - 256, dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError, match="workspace"):
        capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP4, 1, 1, m, k, n, workspace=small)


@pytest.mark.parametrize("kernel", ["stream", "wide", "tile", "tile256", "tile4waves", "tile384", "expanded"])
@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("batch,b_batch,m,k,n", [(1, 1, 256, 128, 256), (1, 1, 300, 96, 288), (2, 1, 130, 160, 96), (1, 1, 288, 224, 96),
                                                 (2, 2, 512, 64, 544), (1, 1, 40, 32, 2080),
                                                 (2, 2, 32, 1024, 224), (3, 1, 24, 768, 160)])
def test_every_kernel_on_every_shape(oracle, kernel, fmt, batch, b_batch, m, k, n, knobs):
    """Each GEMM kernel forced onto shapes it would not be chosen for: ragged row blocks, odd tile counts, one k step,
    more than eight 256-column blocks, shared and per-slice weights, k ranges long enough for the streaming kernels to
    share outputs between workgroups (with batches and ragged column groups); TILE layout in and out, bias and activation."""
    knobs("kernel", "tile" if kernel.startswith("tile") else kernel)
    if kernel == "tile256":
        knobs("block", 256)
    if kernel == "tile4waves":
        knobs("block", 4)
    if kernel == "tile384":                                  # 384-row x 64-column blocks, twelve wavefronts
        knobs("block", 384)
    a_bits = workloads.activations_bf16(m, k, seed=75, batch=batch)
    w = workloads.weights_f32(k, n, seed=76, batch=b_batch)
    words, w_unpacked = pack_weights(oracle, w, fmt)
    a = workloads.bf16_bits_to_f32(a_bits).reshape(batch, m, k)
    w_unpacked = w_unpacked.reshape(b_batch, k, n)
    a_dev = bf16_dev(a_bits).reshape(batch, m, k)
    c = capi.matmul_bfp(a_dev, capi.ROW_MAJOR, words, fmt, batch, b_batch, m, k, n, out_dtype=torch.float32)
    for b in range(batch):
        check_against_reference(c[b].cpu().numpy(), a[b], w_unpacked[b if b_batch > 1 else 0], k, bf16_out=False)
    # TILE layout on both sides gives the same bits as row-major
    c_rm = capi.matmul_bfp(a_dev, capi.ROW_MAJOR, words, fmt, batch, b_batch, m, k, n)
    if m % 32 == 0:                                          # the C ABI takes TILE operands only with whole tiles
        c_tiles = capi.matmul_bfp(capi.tilize(a_dev), capi.TILE, words, fmt, batch, b_batch, m, k, n, c_layout=capi.TILE)
        assert torch.equal(capi.untilize(c_tiles, (batch, m, n)).view(torch.int16), c_rm.view(torch.int16))
    # bias and activation
    bias_bits = workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=77))
    g = capi.matmul_bfp(a_dev, capi.ROW_MAJOR, words, fmt, batch, b_batch, m, k, n, bias=bf16_dev(bias_bits),
                        activation=capi.ACT_RELU, out_dtype=torch.float32)
    want = torch.relu(c + torch.from_numpy(workloads.bf16_bits_to_f32(bias_bits)).cuda())
    assert torch.allclose(g, want, rtol=1e-5, atol=1e-5)


def test_expanded_weights_in_a_caller_workspace(oracle, knobs):
    knobs("kernel", "expanded")
    m, k, n = 512, 128, 160
    a_bits = workloads.activations_bf16(m, k, seed=78)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=79), BFP8)
    need = capi.lib().ttmi_matmul_bfp_workspace_bytes(1, m, k, n, BFP8)
    assert need == (k // 32) * 3 * 4096                      # 2 bytes per weight, 64-column groups
    ws = torch.full((need,), 0x5A, dtype=torch.uint8, device="cuda")
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n, workspace=ws)
    check_against_reference(c.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)
    own = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)
    assert torch.equal(own.view(torch.int16), c.view(torch.int16))
    with pytest.raises(RuntimeError, match="workspace"):
        capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n,
                        workspace=torch.empty(need - 256, dtype=torch.uint8, device="cuda"))


def test_decode_gemm_in_a_hip_graph(oracle):
    """A caller that captures the stream: with its own workspace the call records kernels only (the slots are marked empty by
    a fill kernel, no memset node).  Replayed several times with eager work and synchronisation in between, every replay
    must give the eager result."""
    m, k, n = 32, 2048, 320
    a_bits = workloads.activations_bf16(m, k, seed=90)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=91), BFP8)
    a = bf16_dev(a_bits)
    need = capi.lib().ttmi_matmul_bfp_workspace_bytes(1, m, k, n, BFP8)
    assert need > 0
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    eager = capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n, workspace=ws).clone()
    check_against_reference(eager.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)
    out = torch.zeros(m * n, dtype=torch.bfloat16, device="cuda")
    L = capi.lib()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            capi.check(L.ttmi_matmul_bfp(a.data_ptr(), capi.ROW_MAJOR, words.data_ptr(), BFP8, 1, 1, m, k, n, None, capi.ACT_NONE,
                                         out.data_ptr(), capi.ROW_MAJOR, capi.BFLOAT16, ws.data_ptr(), need, side.cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(4):
        out.zero_()
        ws.fill_(replay)                                        # the workspace may hold anything between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(1, m, n).view(torch.int16), eager.view(torch.int16)), replay
        other = capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)      # eager work between the replays
        assert torch.equal(other.view(torch.int16), eager.view(torch.int16))


@pytest.mark.parametrize("kernel", ["stream", "wide"])
@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_row_exponents_over_the_whole_range(oracle, kernel, fmt, knobs):
    """Weight rows scaled by 2^s, s in [-100, 100], against activation columns scaled by 2^-s: every shared exponent from
    about 20 to 230 occurs, the products stay of order one, and the result must not care (scales are exact powers of two)."""
    knobs("kernel", kernel)
    rng = np.random.default_rng(97)
    m, k, n = 32, 512, 256
    shift = rng.integers(-100, 101, size=k)
    a = workloads.bf16_bits_to_f32(workloads.activations_bf16(m, k, seed=98)) * np.exp2(-shift)[None, :].astype(np.float32)
    w = workloads.weights_f32(k, n, seed=99) * np.exp2(shift)[:, None].astype(np.float32)
    a_bits = workloads.f32_to_bf16_bits_rne(a.astype(np.float32))
    assert np.array_equal(workloads.bf16_bits_to_f32(a_bits), a.astype(np.float32))          # still exact in bf16
    words, w_unpacked = pack_weights(oracle, w.astype(np.float32), fmt)
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n, out_dtype=torch.float32)
    check_against_reference(c.cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k, bf16_out=False)


def test_decode_gemms_on_two_streams_at_once(oracle):
    """Two decode GEMMs, each with a workspace of its own, queued on two streams without waiting for each other: neither
    grid is resident as a whole while the other runs, and the hand-over of partial sums must neither stall nor mix.  Every
    result equals the one computed alone."""
    shapes = [(32, 4096, 1024, BFP8, 92), (32, 2048, 4096, BFP4, 94)]
    L = capi.lib()
    jobs = []
    for m, k, n, fmt, seed in shapes:
        a = bf16_dev(workloads.activations_bf16(m, k, seed=seed))
        words = capi.pack_tensor(fmt, dev(workloads.weights_f32(k, n, seed=seed + 1)))
        need = L.ttmi_matmul_bfp_workspace_bytes(1, m, k, n, fmt)
        assert need > 0
        alone = capi.matmul_bfp(a, capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n).clone()
        jobs.append(dict(m=m, k=k, n=n, fmt=fmt, a=a, words=words, need=need, alone=alone, stream=torch.cuda.Stream(),
                         ws=torch.full((need,), 0x33, dtype=torch.uint8, device="cuda"),
                         outs=[torch.zeros(m * n, dtype=torch.bfloat16, device="cuda") for _ in range(12)]))
    torch.cuda.synchronize()
    for rep in range(12):
        for j in jobs:
            capi.check(L.ttmi_matmul_bfp(j["a"].data_ptr(), capi.ROW_MAJOR, j["words"].data_ptr(), j["fmt"], 1, 1, j["m"], j["k"], j["n"],
                                         None, capi.ACT_NONE, j["outs"][rep].data_ptr(), capi.ROW_MAJOR, capi.BFLOAT16,
                                         j["ws"].data_ptr(), j["need"], j["stream"].cuda_stream))
    torch.cuda.synchronize()
    for j in jobs:
        for rep, out in enumerate(j["outs"]):
            assert torch.equal(out.view(1, j["m"], j["n"]).view(torch.int16), j["alone"].view(torch.int16)), (j["n"], rep)


def test_full_size_decode_gemms_on_three_streams():
    """The same at full size: together the three grids are more than twice what the GPU holds at one time, so workgroups
    of every launch wait for slots while others of the same launch already poll for their partial sums.  That costs time
    (whoever waits, waits for lower workgroup indices only, so it ends), never results."""
    L = capi.lib()
    jobs = []
    for m, k, n, fmt, seed in [(32, 4544, 18176, BFP8, 1), (32, 18176, 4544, BFP8, 2), (32, 4096, 14336, BFP4, 3)]:
        gen = torch.Generator(device="cuda").manual_seed(seed)
        a = capi.tilize(torch.randn(m, k, device="cuda", generator=gen).bfloat16())
        w = capi.pack_tensor(fmt, torch.randn(k, n, device="cuda", generator=gen) * 0.02)
        need = L.ttmi_matmul_bfp_workspace_bytes(1, m, k, n, fmt)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        alone = capi.matmul_bfp(a, capi.TILE, w, fmt, 1, 1, m, k, n, c_layout=capi.TILE).clone()
        jobs.append(dict(m=m, k=k, n=n, fmt=fmt, a=a, w=w, need=need, ws=ws, alone=alone, stream=torch.cuda.Stream(),
                         outs=[torch.empty(m * n, dtype=torch.bfloat16, device="cuda") for _ in range(8)]))
    torch.cuda.synchronize()
    for rep in range(8):
        for j in jobs:
            capi.check(L.ttmi_matmul_bfp(j["a"].data_ptr(), capi.TILE, j["w"].data_ptr(), j["fmt"], 1, 1, j["m"], j["k"], j["n"], None,
                                         capi.ACT_NONE, j["outs"][rep].data_ptr(), capi.TILE, capi.BFLOAT16, j["ws"].data_ptr(), j["need"],
                                         j["stream"].cuda_stream))
    torch.cuda.synchronize()
    for j in jobs:
        again = capi.matmul_bfp(j["a"], capi.TILE, j["w"], j["fmt"], 1, 1, j["m"], j["k"], j["n"], c_layout=capi.TILE)
        want = j["alone"].reshape(-1).view(torch.int16)
        differing = {"alone again": int((again.reshape(-1).view(torch.int16) != want).sum())}
        differing.update({f"launch {rep}": int((out.view(torch.int16) != want).sum()) for rep, out in enumerate(j["outs"])})
        assert not any(differing.values()), (j["n"], differing)


def oracle_unpacked(oracle, fmt, words, k, n, batch=1):
    """The weights as the reference's host unpacker and untilizer give them back (CPU oracle), [batch, k, n] fp32."""
    flat = oracle.unpack_bfp_tiles_into_float_vec(fmt, words.cpu().numpy().view(np.uint32), False)
    return oracle.untilize_nchw_4faces(flat, (1, batch, k, n))[0]


def check_on_gpu(c, a_bits, w_unpacked, k, bf16_out=True):
    """check_against_reference for sizes where the fp64 products are better formed on the GPU: the reference is a float64
    matmul (torch, on the device) of the exact activations with the oracle-unpacked weights; every element is held to the
    stated bound, and the PCC is taken over all of them."""
    a64 = torch.from_numpy(workloads.bf16_bits_to_f32(a_bits)).cuda().double()
    w64 = torch.from_numpy(np.ascontiguousarray(w_unpacked)).cuda().double()
    ref = a64 @ w64
    mag = a64.abs() @ w64.abs()
    bound = (2.0 ** -8 if bf16_out else 2.0 ** -22) * ref.abs() + 2.0 * k * 2.0 ** -24 * mag + 1e-37
    got = c.double()
    worst = float(((got - ref).abs() / bound).max())
    assert worst <= 1.0, f"elementwise bound exceeded by factor {worst}"
    pcc = float(torch.corrcoef(torch.stack([ref.reshape(-1), got.reshape(-1)]))[0, 1])
    assert pcc >= 0.9999, pcc
    return pcc


@pytest.mark.parametrize("layout", [capi.ROW_MAJOR, capi.TILE])
@pytest.mark.parametrize("name,m,k,n,fmt,batch", workloads.DECODE_FALCON + workloads.DECODE_MISTRAL)
def test_decode_shapes_full_size(oracle, name, m, k, n, fmt, batch, layout):
    """Every decode GEMM of the workloads at full size, in both operand layouts (TILE is what ttnn.matmul takes and returns and
    what the benchmark times), every output element against the float64 product with the oracle-unpacked weights."""
    a_bits = workloads.activations_bf16(m, k, seed=80)
    words = capi.pack_tensor(FMT[fmt], dev(workloads.weights_f32(k, n, seed=81)))
    w_unpacked = oracle_unpacked(oracle, FMT[fmt], words, k, n)[0]
    a = bf16_dev(a_bits)
    if layout == capi.TILE:
        c = capi.untilize(capi.matmul_bfp(capi.tilize(a), capi.TILE, words, FMT[fmt], 1, 1, m, k, n, c_layout=capi.TILE), (1, m, n))
    else:
        c = capi.matmul_bfp(a, capi.ROW_MAJOR, words, FMT[fmt], 1, 1, m, k, n)
    pcc = check_against_reference(c.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)
    print(name, "pcc", pcc)


@pytest.mark.parametrize("m,k,n,fmt", [(32, 4096, 16384, "bfp8_b"), (32, 4096, 21760, "bfp4_b"), (256, 4096, 4096, "bfp8_b")])
def test_shapes_whose_collecting_workgroups_come_on_top(oracle, m, k, n, fmt):
    """128 and 170 output groups (and 4 pairs of row bands x 32): one more k range per output fills the places that the
    workgroups which only collect would have been given, so those come on top of a full chip and start late.  Every
    output element against the float64 product with the oracle-unpacked weights."""
    plan = (ctypes.c_uint32 * 4)()
    capi.lib().ttmi_matmul_bfp_plan(1, m, k, n, capi.BFLOAT16, FMT[fmt], capi.BFLOAT16, plan)
    assert plan[0] == 2 and plan[2] > 512, list(plan)                    # 128-column kernel, more workgroups than places
    a_bits = workloads.activations_bf16(m, k, seed=86)
    words = capi.pack_tensor(FMT[fmt], dev(workloads.weights_f32(k, n, seed=87)))
    w_unpacked = oracle_unpacked(oracle, FMT[fmt], words, k, n)[0]
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, FMT[fmt], 1, 1, m, k, n)
    capi.device_status()
    check_on_gpu(c[0], a_bits, w_unpacked, k)


@pytest.mark.parametrize("m", [64, 128 - 3])
@pytest.mark.parametrize("name,k,n,fmt", [("falcon_h_to_4h", 4544, 18176, "bfp8_b"), ("falcon_4h_to_h", 18176, 4544, "bfp8_b"), ("mistral_gate", 4096, 14336, "bfp4_b")])
def test_two_and_four_row_bands_full_size(oracle, name, m, k, n, fmt):
    """64 and 125 rows on the decode shapes (the two-band form of the 128-column kernel: the weights once per 64 rows; 125 rows
    leave the last band ragged), every output element against the float64 product with the oracle-unpacked weights."""
    a_bits = workloads.activations_bf16(m, k, seed=84)
    words = capi.pack_tensor(FMT[fmt], dev(workloads.weights_f32(k, n, seed=85)))
    w_unpacked = oracle_unpacked(oracle, FMT[fmt], words, k, n)[0]
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, FMT[fmt], 1, 1, m, k, n)
    check_on_gpu(c[0], a_bits, w_unpacked, k)
    if m % 32 == 0:
        tiles = capi.matmul_bfp(capi.tilize(bf16_dev(a_bits)), capi.TILE, words, FMT[fmt], 1, 1, m, k, n, c_layout=capi.TILE)
        assert torch.equal(capi.untilize(tiles, (1, m, n)).view(torch.int16), c.view(torch.int16))


@pytest.mark.parametrize("layout", [capi.ROW_MAJOR, capi.TILE])
def test_prefill_shape_full_size_every_row(oracle, layout):
    """[2048,4096] x BFP8 [4096,14336]: all 2048 x 14336 outputs against the float64 product with the weights as the CPU
    oracle unpacks them."""
    name, m, k, n, fmt, _ = workloads.PREFILL[0]
    a_bits = workloads.activations_bf16(m, k, seed=82)
    words = capi.pack_tensor(BFP8, dev(workloads.weights_f32(k, n, seed=83)))
    w_unpacked = oracle_unpacked(oracle, BFP8, words, k, n)[0]
    a = bf16_dev(a_bits)
    if layout == capi.TILE:
        c = capi.untilize(capi.matmul_bfp(capi.tilize(a), capi.TILE, words, BFP8, 1, 1, m, k, n, c_layout=capi.TILE), (1, m, n))
    else:
        c = capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)
    check_on_gpu(c[0], a_bits, w_unpacked, k)


def test_bert_like_bmm_full_size_every_slice(oracle):
    name, m, k, n, fmt, batch = workloads.PREFILL[1]
    a_bits = workloads.activations_bf16(m, k, seed=85, batch=batch)
    w = workloads.weights_f32(k, n, seed=86, batch=batch)
    words, w_unpacked = pack_weights(oracle, w, BFP8)
    a = bf16_dev(a_bits)
    c = capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, batch, batch, m, k, n)
    c_tiles = capi.untilize(capi.matmul_bfp(capi.tilize(a.reshape(batch, m, k)), capi.TILE, words, BFP8, batch, batch, m, k, n, c_layout=capi.TILE), (batch, m, n))
    assert torch.equal(c_tiles.view(torch.int16), c.view(torch.int16))
    for b in range(batch):
        check_on_gpu(c[b], a_bits.reshape(batch, m, k)[b], w_unpacked[b], k)


# ---- rows at the ends of the exponent range ------------------------------------------------------------------------------
def assemble_tiles(fmt, exps, codes):
    """Packed tiles from shared exponents [K, N / 16] and codes [K, N] (sign | mantissa), laid out as
    tt_metal/common/bfloat8.hpp:102-173 does: 64 exponent bytes (face, row), then the faces row by row, element 0 in the
    low bits; tile (kt, nt) at kt * Nt + nt.  Lets a test hold exponent bytes that no packer writes next to given codes."""
    k, n = codes.shape
    kt, nt = k // 32, n // 32
    tile_bytes = 1088 if fmt == BFP8 else 576
    out = np.zeros((kt, nt, tile_bytes), dtype=np.uint8)
    for face in range(4):
        fr, fc = face >> 1, face & 1
        e = exps.reshape(kt, 2, 16, nt, 2)[:, fr, :, :, fc]                       # [kt, 16, nt]
        out[:, :, face * 16:(face + 1) * 16] = e.transpose(0, 2, 1)
        block = codes.reshape(kt, 2, 16, nt, 2, 16)[:, fr, :, :, fc, :].transpose(0, 2, 1, 3)       # [kt, nt, 16 rows, 16 columns]
        if fmt == BFP8:
            out[:, :, 64 + face * 256:64 + (face + 1) * 256] = block.reshape(kt, nt, 256)
        else:
            out[:, :, 64 + face * 128:64 + (face + 1) * 128] = (block[..., 0::2] | (block[..., 1::2] << 4)).reshape(kt, nt, 128)
    return np.ascontiguousarray(out).reshape(-1).view(np.uint32)


EDGE_KERNELS = [("wide", 32, None), ("wide", 64, None), ("stream", 64, None), ("tile", 256, 128), ("tile", 256, 256), ("tile", 256, 4), ("tile", 384, 384), ("expanded", 512, None)]


@pytest.mark.parametrize("kernel,m,block", EDGE_KERNELS)
@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_rows_at_the_ends_of_the_exponent_range(oracle, kernel, m, block, fmt, knobs):
    """What every GEMM kernel does with shared exponents that ordinary weights never have, pinned kernel by kernel:
      E = 0     (fp32 subnormal sources)  the row is read with the scale of E = 1, the IEEE convention for a zero exponent
                field; the same in every kernel
      E = 247   the largest exponent every kernel takes exactly
      E = 254   exact in the streaming kernels (M < 128) where they take the weights in hidden-one form; in the tiled and
                expanding kernels, and in the two-band form of the 128-column kernel (single exact operands), the operand,
                mantissa x 2^(E - 127), overflows for mantissas >= 2: those columns come out non-finite
      E = 255   (Inf / NaN sources) the 16 columns that share the exponent are non-finite, all others are untouched
    Expected values are formed here from codes and exponents directly: sign x mantissa x 2^(max(E, 1) - 127 - (W - 1))."""
    knobs("kernel", kernel)
    if block:
        knobs("block", block)
    w_bits = 7 if fmt == BFP8 else 3
    rng = np.random.default_rng(130 + m)
    k, n = 128, 128
    exps = rng.integers(118, 131, size=(k, n // 16)).astype(np.uint8)
    codes = rng.integers(0, 1 << (w_bits + 1), size=(k, n)).astype(np.uint8)
    a = rng.standard_normal((m, k)).astype(np.float32)
    exps[5, :], a[:, 5] = 0, a[:, 5] * 2.0 ** 124            # products of order one: 2^124 x mantissa x 2^(1 - 133)
    exps[40, :], a[:, 40] = 247, a[:, 40] * 2.0 ** -120
    exps[77, :], a[:, 77] = 254, a[:, 77] * 2.0 ** -125
    exps[100, 3] = 255
    a_bits = workloads.f32_to_bf16_bits_rne(a)
    a64 = workloads.bf16_bits_to_f32(a_bits).astype(np.float64)
    mant = (codes & ((1 << w_bits) - 1)).astype(np.float64)
    sign = np.where(codes >> w_bits, -1.0, 1.0)
    e_eff = np.maximum(np.repeat(exps, 16, axis=1).astype(np.int64), 1)
    w64 = sign * mant * np.exp2((e_eff - 127 - (w_bits - 1)).astype(np.float64))
    w64[100, 48:64] = 0.0                                   # not part of any expectation: those columns must be non-finite
    words = torch.from_numpy(assemble_tiles(fmt, exps, codes).view(np.int32)).cuda()
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n, out_dtype=torch.float32)[0].cpu().numpy().astype(np.float64)
    ref = a64 @ w64
    bound = 2.0 ** -22 * np.abs(ref) + 2.0 * k * 2.0 ** -24 * (np.abs(a64) @ (np.abs(w64) + np.exp2((e_eff - 127).astype(np.float64)))) + 1e-37
    poisoned = np.zeros(n, dtype=bool)
    poisoned[48:64] = True                                   # E = 255
    if kernel in ("tile", "expanded") or (kernel == "wide" and m > 32):
        poisoned |= (codes[77] & ((1 << w_bits) - 1)) >= 2   # E = 254: mantissa x 2^127 overflows
    assert not np.isfinite(c[:, poisoned]).any()
    ok = ~poisoned
    assert np.isfinite(c[:, ok]).all()
    assert np.all(np.abs(c[:, ok] - ref[:, ok]) <= bound[:, ok]), float(np.max(np.abs(c[:, ok] - ref[:, ok]) / bound[:, ok]))
    # the rows at the ends carry weight in the sums: without them the check above would fail
    without = ref - a64[:, [5, 40, 77]] @ w64[[5, 40, 77]]
    assert np.max(np.abs(without[:, ok] - ref[:, ok]) / bound[:, ok]) > 100.0


@pytest.mark.parametrize("kernel,m", [("wide", 32), ("stream", 64)])
def test_a_wait_that_gives_up_is_reported_and_leaves_later_calls_correct(oracle, kernel, m, knobs):
    """Forced from the host: producers keep their partial sums to themselves and the bounded wait is cut to a few polls,
    so every collector gives up (every kernel still runs to its end).  The launch raises the device's error word, the
    next call reports TTMI_ERR_HIP, and the call after that — on slots that the library refills — is correct again."""
    k, n = 2048, 256
    a_bits = workloads.activations_bf16(m, k, seed=120)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=121), BFP8)
    a = bf16_dev(a_bits)
    knobs("kernel", kernel)
    good = capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)
    torch.cuda.synchronize()
    capi.device_status()                                                # nothing to report
    knobs("drop_partial_sums", 1)
    knobs("spin_limit", 3)
    capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)     # outputs shared between workgroups: the waits give up
    torch.cuda.synchronize()
    knobs("drop_partial_sums", 0)
    knobs("spin_limit", 1 << 20)
    with pytest.raises(RuntimeError, match="gave up waiting"):
        capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)
    capi.device_status()                                                # reported once, then clear
    again = capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)
    torch.cuda.synchronize()
    capi.device_status()
    assert torch.equal(again.view(torch.int16), good.view(torch.int16))
    check_against_reference(again.float().cpu().numpy()[0], workloads.bf16_bits_to_f32(a_bits), w_unpacked, k)


def test_a_wait_that_gives_up_is_raised_where_the_result_is_read(oracle, knobs):
    """The same forced give-up through the TT-NN surface: the matmul returns (its kernels run to their end), and the call that
    brings the bad result to the host — ttnn.to_torch, ttnn.from_device, Tensor.cpu — raises instead of handing it over."""
    import ttnn

    m, k, n = 32, 2048, 256
    torch.manual_seed(7)
    device = ttnn.open_device(0)
    x = torch.randn(1, 1, m, k).to(torch.bfloat16)
    tx = ttnn.from_torch(x, dtype=ttnn.bfloat16, layout=ttnn.TILE_LAYOUT, device=device)
    tw = ttnn.from_torch(torch.randn(1, 1, k, n) * 0.02, dtype=ttnn.bfloat8_b, layout=ttnn.TILE_LAYOUT, device=device)
    knobs("kernel", "wide")
    good = ttnn.to_torch(ttnn.matmul(tx, tw))
    for read in (ttnn.to_torch, ttnn.from_device, lambda t: t.cpu()):
        knobs("drop_partial_sums", 1)
        knobs("spin_limit", 3)
        bad = ttnn.matmul(tx, tw)
        torch.cuda.synchronize()
        knobs("drop_partial_sums", 0)
        knobs("spin_limit", 1 << 20)
        with pytest.raises(RuntimeError, match="gave up waiting"):
            read(bad)
        assert torch.equal(ttnn.to_torch(ttnn.matmul(tx, tw)), good)        # reported once; the slots are refilled


def test_library_scratch_can_be_released(oracle, test_library):
    """ttmi_release_scratch frees what the library holds on the device (buffers per stream, and those it had outgrown) once
    the device is idle; the next call allocates again and gives the same bits."""
    m, k, n = 32, 4096, 512
    a = bf16_dev(workloads.activations_bf16(m, k, seed=124))
    words, _ = pack_weights(oracle, workloads.weights_f32(k, n, seed=125), BFP8)
    streams = [torch.cuda.Stream() for _ in range(3)]
    outs = []
    for stream in streams:
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            outs.append(capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n))
    torch.cuda.synchronize()
    L = capi.lib()
    L.ttmi_test_allocations.restype = ctypes.c_uint64
    free_before, made_before = torch.cuda.mem_get_info()[0], L.ttmi_test_allocations()
    freed = capi.release_scratch()
    assert freed >= 3 * capi.lib().ttmi_matmul_bfp_workspace_bytes(1, m, k, n, BFP8) > 0       # a buffer per stream, at least
    assert torch.cuda.mem_get_info()[0] >= free_before + freed // 2                              # back with the device (allocation granularity aside)
    assert capi.release_scratch() == 0
    with torch.cuda.stream(streams[0]):
        again = capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n)
    torch.cuda.synchronize()
    capi.device_status()
    assert L.ttmi_test_allocations() > made_before
    assert all(torch.equal(again.view(torch.int16), c.view(torch.int16)) for c in outs)


def test_library_scratch_is_per_stream(oracle):
    """Without a caller workspace every stream gets slots of its own, so decode GEMMs issued on two streams at once do not
    share partial sums (the same two calls on one stream share a buffer and run in order)."""
    m, k, n = 32, 4096, 512
    a_bits = workloads.activations_bf16(m, k, seed=122)
    words, w_unpacked = pack_weights(oracle, workloads.weights_f32(k, n, seed=123), BFP8)
    a = bf16_dev(a_bits)
    want = capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n).clone()
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    results = [[], []]
    for rep in range(20):
        for s, stream in enumerate(streams):
            with torch.cuda.stream(stream):
                results[s].append(capi.matmul_bfp(a, capi.ROW_MAJOR, words, BFP8, 1, 1, m, k, n))
    torch.cuda.synchronize()
    capi.device_status()
    for per_stream in results:
        for c in per_stream:
            assert torch.equal(c.view(torch.int16), want.view(torch.int16))


def test_library_slots_beyond_the_first_launch_are_empty_too():
    """The library's slot buffer grows geometrically, so a launch may find room for more slots than any launch before it
    has used: those must be empty as well (the whole buffer is filled when it is new, not only what the first launch
    needs).  Three GEMMs on a new stream whose slot needs are 64, 80 and 112 workgroups x 16 KB: the second makes the
    buffer grow to 2 MB, the third fits without growing.  Each is compared with the same GEMM on a caller's workspace,
    which is filled on every call."""
    L = capi.lib()
    stream = torch.cuda.Stream()
    m, k = 32, 2048
    for groups in (8, 10, 14):
        n = 128 * groups
        gen = torch.Generator(device="cuda").manual_seed(groups)
        a = capi.tilize(torch.randn(m, k, device="cuda", generator=gen).bfloat16())
        w = capi.pack_tensor(BFP8, torch.randn(k, n, device="cuda", generator=gen) * 0.02)
        need = L.ttmi_matmul_bfp_workspace_bytes(1, m, k, n, BFP8)
        assert need == groups * 8 * 16384
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        want = torch.empty(m * n, dtype=torch.bfloat16, device="cuda")
        got = torch.empty(m * n, dtype=torch.bfloat16, device="cuda")
        torch.cuda.synchronize()
        args = (a.data_ptr(), capi.TILE, w.data_ptr(), BFP8, 1, 1, m, k, n, None, capi.ACT_NONE)
        capi.check(L.ttmi_matmul_bfp(*args, want.data_ptr(), capi.TILE, capi.BFLOAT16, ws.data_ptr(), need, stream.cuda_stream))
        capi.check(L.ttmi_matmul_bfp(*args, got.data_ptr(), capi.TILE, capi.BFLOAT16, None, 0, stream.cuda_stream))
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), groups


@pytest.mark.parametrize("out_fmt", [BFP8, BFP4])
@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("batch,m,k,n", [(1, 32, 64, 128), (1, 32, 2048, 256), (1, 32, 4096, 96), (2, 32, 1024, 2080), (1, 64, 512, 160),
                                         (1, 256, 128, 256), (1, 512, 64, 160)])
def test_block_float_output(oracle, out_fmt, fmt, batch, m, k, n):
    """Output dtype BFLOAT8_B / BFLOAT4_B (TILE layout): the words are those that packing the bf16 output of the same GEMM
    gives (ttmi_typecast_tiles, itself pinned against the oracle's packer) — packed in the epilogue of whichever kernel the
    shape goes to, stored directly and through the hand-over of partial sums, with a column group that is not full — and
    unpack to the oracle's unpacking of those words."""
    a_bits = workloads.activations_bf16(m, k, seed=400, batch=batch)
    words, _ = pack_weights(oracle, workloads.weights_f32(k, n, seed=401), fmt)
    a_tiles = capi.tilize(bf16_dev(a_bits).reshape(batch, m, k))
    bias_bits = workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=402))
    for kwargs in ({}, {"bias": bf16_dev(bias_bits), "activation": capi.ACT_GELU}):
        dense = capi.matmul_bfp(a_tiles, capi.TILE, words, fmt, batch, 1, m, k, n, c_layout=capi.TILE, **kwargs)
        want = capi.typecast_tiles(dense, capi.BFLOAT16, out_fmt)
        got = capi.matmul_bfp(a_tiles, capi.TILE, words, fmt, batch, 1, m, k, n, c_layout=capi.TILE, out_bfp=out_fmt, **kwargs)
        assert torch.equal(got, want)
    host = oracle.pack_fp32_vec_as_bfp_tiles(out_fmt, dense.float().cpu().numpy().reshape(-1), False)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), host)
    with pytest.raises(RuntimeError, match="TILE layout"):
        capi.check(capi.lib().ttmi_matmul_bfp(a_tiles.data_ptr(), capi.TILE, words.data_ptr(), fmt, batch, 1, m, k, n, None, 0, got.data_ptr(),
                                              capi.ROW_MAJOR, out_fmt, None, 0, None))


@pytest.mark.parametrize("out_fmt", [BFP8, BFP4])
@pytest.mark.parametrize("kernel", ["wide", "tile", "tile256", "tile4waves", "tile384", "expanded"])
@pytest.mark.parametrize("batch,b_batch,m,k,n", [(2, 2, 384, 96, 288), (1, 1, 128, 1024, 96), (3, 1, 64, 2048, 160)])
def test_every_kernel_packs_a_block_float_output_in_its_epilogue(oracle, out_fmt, kernel, batch, b_batch, m, k, n, knobs):
    """No kernel leaves a block-float output to a second launch: forced onto one shape after the other (ragged column groups,
    batches, shared outputs), each writes the words that packing its own bf16 output gives, and those are the oracle's."""
    knobs("kernel", "tile" if kernel.startswith("tile") else kernel)
    if kernel != "tile" and kernel.startswith("tile"):
        knobs("block", {"tile256": 256, "tile4waves": 4, "tile384": 384}[kernel])
    a_bits = workloads.activations_bf16(m, k, seed=410, batch=batch)
    words, _ = pack_weights(oracle, workloads.weights_f32(k, n, seed=411, batch=b_batch), BFP8)
    a_tiles = capi.tilize(bf16_dev(a_bits).reshape(batch, m, k))
    bias = bf16_dev(workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=412)))
    dense = capi.matmul_bfp(a_tiles, capi.TILE, words, BFP8, batch, b_batch, m, k, n, c_layout=capi.TILE, bias=bias, activation=capi.ACT_SILU)
    got = capi.matmul_bfp(a_tiles, capi.TILE, words, BFP8, batch, b_batch, m, k, n, c_layout=capi.TILE, out_bfp=out_fmt, bias=bias, activation=capi.ACT_SILU)
    host = oracle.pack_fp32_vec_as_bfp_tiles(out_fmt, dense.float().cpu().numpy().reshape(-1), False)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), host)


@pytest.mark.parametrize("batch,b_batch,m,k,n", [(1, 1, 32, 64, 64), (1, 1, 32, 4544, 256), (2, 2, 40, 160, 96), (3, 1, 300, 96, 288), (1, 1, 512, 256, 544)])
def test_bf16_weights(batch, b_batch, m, k, n):
    """Two bf16 operands (ttmi_matmul_bf16): weights in TILE layout, re-laid-out and multiplied by the bf16 GEMM of the
    expanding path; against a float64 matmul of the same values with the bound of the block-float GEMMs; TILE and
    row-major activations give the same bits; bias and activation; block-float output."""
    a_bits = workloads.activations_bf16(m, k, seed=500, batch=batch)
    w_bits = workloads.f32_to_bf16_bits_rne(workloads.weights_f32(k, n, seed=501, batch=b_batch))
    a = workloads.bf16_bits_to_f32(a_bits).reshape(batch, m, k)
    w = workloads.bf16_bits_to_f32(w_bits).reshape(b_batch, k, n)
    a_dev = bf16_dev(a_bits).reshape(batch, m, k)
    w_tiles = capi.tilize(bf16_dev(w_bits).reshape(b_batch, k, n))
    c = capi.matmul_bf16(a_dev, capi.ROW_MAJOR, w_tiles, batch, b_batch, m, k, n, out_dtype=torch.float32)
    for b in range(batch):
        check_against_reference(c[b].cpu().numpy(), a[b], w[b if b_batch > 1 else 0], k, bf16_out=False)
    c16 = capi.matmul_bf16(a_dev, capi.ROW_MAJOR, w_tiles, batch, b_batch, m, k, n)
    for b in range(batch):
        check_against_reference(c16[b].float().cpu().numpy(), a[b], w[b if b_batch > 1 else 0], k)
    if m % 32 == 0:
        tiles = capi.matmul_bf16(capi.tilize(a_dev), capi.TILE, w_tiles, batch, b_batch, m, k, n, c_layout=capi.TILE)
        assert torch.equal(capi.untilize(tiles, (batch, m, n)).view(torch.int16), c16.view(torch.int16))
    bias_bits = workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=502))
    g = capi.matmul_bf16(a_dev, capi.ROW_MAJOR, w_tiles, batch, b_batch, m, k, n, bias=bf16_dev(bias_bits), activation=capi.ACT_RELU, out_dtype=torch.float32)
    assert torch.allclose(g, torch.relu(c + torch.from_numpy(workloads.bf16_bits_to_f32(bias_bits)).cuda()), rtol=1e-5, atol=1e-5)
    need = capi.lib().ttmi_matmul_bf16_workspace_bytes(b_batch, k, n)
    assert need == b_batch * (k // 32) * ((n // 32 + 1) // 2) * 4096
    ws = torch.full((need,), 0x5A, dtype=torch.uint8, device="cuda")
    again = capi.matmul_bf16(a_dev, capi.ROW_MAJOR, w_tiles, batch, b_batch, m, k, n, workspace=ws)
    assert torch.equal(again.view(torch.int16), c16.view(torch.int16))


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("kernel", ["wide", "wide two bands", "stream", "tile", "expanded"])
def test_face_rows_with_outliers(oracle, fmt, kernel, knobs):
    """Weights whose face rows mix magnitudes over 40 binades (the stress mixture, x 50): for the kernels that multiply by
    the expanded weights the error stays within the fp32 accumulation bound on |A| . |W|; the streaming kernels add and
    subtract the face row's power of two with every weight (hi - lo), so their accumulation error is relative to that
    power of two - at most 2^-16 of the row's own quantisation step per product - and an output next to an outlier can
    leave the |W| bound while the sum over all outputs is as accurate as before (relative rms error below 1e-6)."""
    m, k, n = (64 if kernel == "wide two bands" else 32), 256, 384
    w = np.ascontiguousarray(workloads.stress_mixture((1, 1, k, n), seed=3)[0, 0] * 50.0)
    words, w_ref = pack_weights(oracle, w, fmt)
    a_bits = workloads.activations_bf16(m, k, seed=4)
    a = workloads.bf16_bits_to_f32(a_bits)
    knobs("kernel", kernel.split()[0])
    c = capi.matmul_bfp(bf16_dev(a_bits), capi.ROW_MAJOR, words, fmt, 1, 1, m, k, n, out_dtype=torch.float32)[0].cpu().numpy()
    # hidden-one form: the 64-column kernel and the 128-column kernel with one band
    check_against_reference(c, a, w_ref, k, bf16_out=False, face_row_scale=kernel in ("wide", "stream"))
    ref = a.astype(np.float64) @ w_ref.astype(np.float64)
    assert np.sqrt(((c - ref) ** 2).mean() / (ref ** 2).mean()) < 1e-6


@pytest.mark.parametrize("fmt,batch,b_batch,m,k,n", [
    (BFP8, 1, 1, 32, 4544, 4608), (BFP8, 1, 1, 32, 1024, 288), (BFP4, 1, 1, 32, 4096, 14336), (BFP4, 2, 2, 32, 2048, 160),
    (BFP8, 3, 1, 32, 512, 96), (BFP4, 1, 1, 32, 14336, 4096), (BFP8, 1, 1, 32, 64, 32)])
def test_block_float_activations_are_expanded_inside_the_streaming_kernel(oracle, fmt, batch, b_batch, m, k, n):
    """ttmi_matmul_bfp_ab: packed BFLOAT8_B activations go into the kernel that streams the weights as they are (one band of
    rows per batch slice: BFP4_B and BFP8_B weights, batches, shared outputs, ragged column groups).  The result is bit for bit
    what expanding them first (ttmi_typecast_tiles) and calling ttmi_matmul_bfp gives — bf16, fp32 and block-float outputs,
    bias and activation — and it meets the element-wise bound against a float64 product of the oracle-unpacked operands."""
    L = capi.lib()
    assert L.ttmi_matmul_bfp_ab_supported(batch, m, k, n, BFP8, fmt) == 1
    a_f32 = workloads.bf16_bits_to_f32(workloads.activations_bf16(m, k, seed=600, batch=batch)).reshape(batch, m, k)
    a_f32 = a_f32 * np.exp2(np.arange(m) % 7 - 3).astype(np.float32)[None, :, None]       # face rows of different exponents
    a_words = capi.pack_tensor(BFP8, dev(a_f32))
    a_host = oracle.from_torch_bfp_tiles(BFP8, a_f32)
    assert np.array_equal(a_words.cpu().numpy().view(np.uint32), a_host)
    a_q = oracle.to_torch_bfp_tiles(BFP8, a_host, a_f32.shape)
    w = workloads.weights_f32(k, n, seed=601, batch=b_batch)
    words, w_q = pack_weights(oracle, w, fmt)
    w_q = w_q.reshape(b_batch, k, n)
    a_tiles = capi.typecast_tiles(a_words, BFP8, capi.BFLOAT16)
    bias = bf16_dev(workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=602)))
    for kwargs in ({}, {"out_dtype": torch.float32}, {"bias": bias, "activation": capi.ACT_GELU}, {"c_layout": capi.TILE, "out_bfp": BFP8}):
        kwargs = {"c_layout": capi.TILE, **kwargs}
        two = capi.matmul_bfp(a_tiles, capi.TILE, words, fmt, batch, b_batch, m, k, n, **kwargs)
        one = capi.matmul_bfp_ab(a_words, BFP8, words, fmt, batch, b_batch, m, k, n, **kwargs)
        assert torch.equal(one.view(torch.int16), two.view(torch.int16)), kwargs
    c = capi.matmul_bfp_ab(a_words, BFP8, words, fmt, batch, b_batch, m, k, n, out_dtype=torch.float32)
    capi.device_status()
    for b in range(batch):
        check_against_reference(c[b].cpu().numpy(), a_q[b], w_q[b if b_batch > 1 else 0], k, bf16_out=False, face_row_scale=True)


def test_block_float_activations_where_no_kernel_takes_them():
    """Shapes that go to the MFMA-bound kernels, and BFLOAT4_B activations: refused with TTMI_ERR_UNSUPPORTED before any
    launch; the host layer expands such activations first (tests/test_gpu_ttnn.py multiplies two BFLOAT8_B tensors)."""
    L = capi.lib()
    one = ctypes.c_void_p(256)
    assert L.ttmi_matmul_bfp_ab_supported(1, 2048, 4096, 14336, BFP8, BFP8) == 0
    assert L.ttmi_matmul_bfp_ab_supported(12, 384, 1024, 1024, BFP8, BFP8) == 0
    assert L.ttmi_matmul_bfp_ab_supported(1, 32, 4096, 4096, BFP4, BFP8) == 0
    assert L.ttmi_matmul_bfp_ab_supported(1, 40, 4096, 4096, BFP8, BFP8) == 0           # whole tiles of A only
    assert L.ttmi_matmul_bfp_ab_supported(1, 64, 4096, 4096, BFP8, BFP8) == 0           # one band of rows only
    assert L.ttmi_matmul_bfp_ab(one, BFP8, one, BFP8, 1, 1, 64, 4096, 4096, None, 0, one, capi.TILE, capi.BFLOAT16, None, 0, None) == 3
    assert L.ttmi_matmul_bfp_ab(one, BFP8, one, BFP8, 1, 1, 2048, 4096, 14336, None, 0, one, capi.TILE, capi.BFLOAT16, None, 0, None) == 3
    assert b"ttmi_typecast_tiles" in L.ttmi_last_error()
    assert L.ttmi_matmul_bfp_ab(one, BFP4, one, BFP8, 1, 1, 32, 4096, 4096, None, 0, one, capi.TILE, capi.BFLOAT16, None, 0, None) == 3
    assert L.ttmi_matmul_bfp_ab(one, capi.BFLOAT16, one, BFP8, 1, 1, 32, 4096, 4096, None, 0, one, capi.TILE, capi.BFLOAT16, None, 0, None) == 1
    assert L.ttmi_matmul_bfp_ab(one, BFP8, one, BFP8, 1, 1, 40, 4096, 4096, None, 0, one, capi.ROW_MAJOR, capi.BFLOAT16, None, 0, None) == 1
