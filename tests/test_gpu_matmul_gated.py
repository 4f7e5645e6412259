"""ttmi_matmul_bfp_gated on a real MI355X: act(A . W_gate + bias) * (A . W_up) in one launch, against a float64 evaluation
of the same expression on oracle-unpacked weights and against the three launches it replaces (two GEMMs and ttnn.mul)."""
import numpy as np
import pytest
import torch

from ttmi import capi, workloads

from test_gpu_matmul import BFP4, BFP8, bf16_dev, comp_pcc, dev, oracle_unpacked, pack_weights

pytestmark = pytest.mark.gpu

ACTS = {
    capi.ACT_NONE: lambda x: x,
    capi.ACT_RELU: lambda x: np.maximum(x, 0.0),
    capi.ACT_SILU: lambda x: x / (1.0 + np.exp(-x)),
}


def check_gated(got_f32, a_f32, wg_f32, wu_f32, k, act, bias_f32=None, bf16_out=True):
    """|c - ref| <= 2^-8 |ref| (bf16 output rounding; 2^-22 for fp32 output) + what the fp32 accumulation errors of the two
    GEMMs can do to the product: |up| x 1.1 x e_gate (the activations used here have slope <= 1.1) + |act(gate)| x e_up,
    with e = 2 K 2^-24 (|A| . |W|) as for the plain GEMM; PCC >= 0.9999."""
    a64, wg64, wu64 = a_f32.astype(np.float64), wg_f32.astype(np.float64), wu_f32.astype(np.float64)
    g, u = a64 @ wg64, a64 @ wu64
    if bias_f32 is not None:
        g = g + bias_f32.astype(np.float64)
    e_g = 2.0 * k * 2.0 ** -24 * (np.abs(a64) @ np.abs(wg64))
    e_u = 2.0 * k * 2.0 ** -24 * (np.abs(a64) @ np.abs(wu64))
    ref = ACTS[act](g) * u
    bound = (2.0 ** -8 if bf16_out else 2.0 ** -22) * np.abs(ref) + 1.1 * np.abs(u) * e_g + np.abs(ACTS[act](g)) * e_u + e_g * e_u + 1e-37
    got = got_f32.astype(np.float64)
    worst = float(np.max(np.abs(got - ref) / bound))
    assert worst <= 1.0, f"elementwise bound exceeded by factor {worst}"
    assert comp_pcc(ref, got) >= 0.9999


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
@pytest.mark.parametrize("act", [capi.ACT_SILU, capi.ACT_NONE, capi.ACT_RELU])
@pytest.mark.parametrize("m,k,n", [(32, 64, 128), (32, 1024, 256), (20, 2048, 96), (32, 32, 2080), (7, 4096, 160)])
def test_gated_small_shapes(oracle, fmt, act, m, k, n):
    """One k step, k ranges shared between workgroups (2048 and 4096 rows of the weights on two or three column groups),
    ragged rows, a column group that is not full, more column groups than k ranges."""
    a_bits = workloads.activations_bf16(m, k, seed=300)
    gate_words, gate = pack_weights(oracle, workloads.weights_f32(k, n, seed=301), fmt)
    up_words, up = pack_weights(oracle, workloads.weights_f32(k, n, seed=302), fmt)
    a = workloads.bf16_bits_to_f32(a_bits)
    c = capi.matmul_bfp_gated(bf16_dev(a_bits), capi.ROW_MAJOR, gate_words, up_words, fmt, 1, 1, m, k, n, activation=act, out_dtype=torch.float32)
    check_gated(c[0].cpu().numpy(), a, gate, up, k, act, bf16_out=False)
    c16 = capi.matmul_bfp_gated(bf16_dev(a_bits), capi.ROW_MAJOR, gate_words, up_words, fmt, 1, 1, m, k, n, activation=act)
    check_gated(c16[0].float().cpu().numpy(), a, gate, up, k, act)


@pytest.mark.parametrize("fmt", [BFP8, BFP4])
def test_gated_layouts_bias_batches_and_workspace(oracle, fmt):
    """TILE layout in and out gives the bits of the row-major call; a bias goes onto the gate before the activation;
    per-slice and shared weights; a caller's workspace of the stated size, full of anything, gives the same bits."""
    batch, m, k, n = 2, 32, 1536, 224
    a_bits = workloads.activations_bf16(m, k, seed=310, batch=batch)
    a = workloads.bf16_bits_to_f32(a_bits).reshape(batch, m, k)
    a_dev = bf16_dev(a_bits).reshape(batch, m, k)
    bias_bits = workloads.f32_to_bf16_bits_rne(workloads.normal_tensor((n,), seed=313))
    bias = workloads.bf16_bits_to_f32(bias_bits)
    for b_batch in (1, 2):
        gate_words, gate = pack_weights(oracle, workloads.weights_f32(k, n, seed=311, batch=b_batch), fmt)
        up_words, up = pack_weights(oracle, workloads.weights_f32(k, n, seed=312, batch=b_batch), fmt)
        gate, up = gate.reshape(b_batch, k, n), up.reshape(b_batch, k, n)
        c = capi.matmul_bfp_gated(a_dev, capi.ROW_MAJOR, gate_words, up_words, fmt, batch, b_batch, m, k, n, bias=bf16_dev(bias_bits))
        for b in range(batch):
            s = b if b_batch > 1 else 0
            check_gated(c[b].float().cpu().numpy(), a[b], gate[s], up[s], k, capi.ACT_SILU, bias_f32=bias)
        tiles = capi.matmul_bfp_gated(capi.tilize(a_dev), capi.TILE, gate_words, up_words, fmt, batch, b_batch, m, k, n,
                                      bias=bf16_dev(bias_bits), c_layout=capi.TILE)
        assert torch.equal(capi.untilize(tiles, (batch, m, n)).view(torch.int16), c.view(torch.int16))
        need = capi.lib().ttmi_matmul_bfp_gated_workspace_bytes(batch, m, k, n, fmt)
        assert need > 0 and need % (2 * 16384) == 0
        ws = torch.full((need,), 0x5A, dtype=torch.uint8, device="cuda")
        again = capi.matmul_bfp_gated(a_dev, capi.ROW_MAJOR, gate_words, up_words, fmt, batch, b_batch, m, k, n, bias=bf16_dev(bias_bits), workspace=ws)
        assert torch.equal(again.view(torch.int16), c.view(torch.int16))
        with pytest.raises(RuntimeError, match="workspace"):
            capi.matmul_bfp_gated(a_dev, capi.ROW_MAJOR, gate_words, up_words, fmt, batch, b_batch, m, k, n, workspace=ws[: need - 256])


@pytest.mark.parametrize("workgroups", [64, 200, 512, 1000])
def test_gated_any_number_of_workgroups_gives_the_same_result(oracle, workgroups, knobs):
    m, k, n = 32, 2048, 384
    a_bits = workloads.activations_bf16(m, k, seed=320)
    gate_words, _ = pack_weights(oracle, workloads.weights_f32(k, n, seed=321), BFP4)
    up_words, _ = pack_weights(oracle, workloads.weights_f32(k, n, seed=322), BFP4)
    want = capi.matmul_bfp_gated(bf16_dev(a_bits), capi.ROW_MAJOR, gate_words, up_words, BFP4, 1, 1, m, k, n)
    knobs("workgroups", workgroups)
    got = capi.matmul_bfp_gated(bf16_dev(a_bits), capi.ROW_MAJOR, gate_words, up_words, BFP4, 1, 1, m, k, n)
    # the k ranges differ, so the fp32 sums are formed in another order: equal within the accumulation error, not in bits
    assert torch.allclose(got.float(), want.float(), rtol=2.0 ** -7, atol=1e-3)


def test_gated_mistral_mlp_shape_full_size(oracle):
    """silu(x w1) * (x w3) of a Mistral-7B layer at M = 32 (BFP4_B [4096, 14336] twice) in TILE layout, every element held
    to the bound against oracle-unpacked weights, and against the three launches it replaces."""
    m, k, n = 32, 4096, 14336
    a_bits = workloads.activations_bf16(m, k, seed=330)
    a = workloads.bf16_bits_to_f32(a_bits)
    gate_words = capi.pack_tensor(BFP4, dev(workloads.weights_f32(k, n, seed=331)))
    up_words = capi.pack_tensor(BFP4, dev(workloads.weights_f32(k, n, seed=332)))
    gate, up = oracle_unpacked(oracle, BFP4, gate_words, k, n)[0], oracle_unpacked(oracle, BFP4, up_words, k, n)[0]
    a_tiles = capi.tilize(bf16_dev(a_bits))
    fused = capi.matmul_bfp_gated(a_tiles, capi.TILE, gate_words, up_words, BFP4, 1, 1, m, k, n, c_layout=capi.TILE)
    check_gated(capi.untilize(fused, (m, n)).float().cpu().numpy(), a, gate, up, k, capi.ACT_SILU)
    h1 = capi.matmul_bfp(a_tiles, capi.TILE, gate_words, BFP4, 1, 1, m, k, n, activation=capi.ACT_SILU, c_layout=capi.TILE)
    h3 = capi.matmul_bfp(a_tiles, capi.TILE, up_words, BFP4, 1, 1, m, k, n, c_layout=capi.TILE)
    three = capi.eltwise(capi.OP_MUL, h1, h3)
    # the three launches round to bf16 three times (2^-9 relative each), the fused one once
    worst = float(((fused.float() - three.float()).abs() / (three.float().abs() + 1e-3)).max())
    assert worst <= 2.0 ** -6, worst


@pytest.mark.parametrize("out_fmt", [BFP8, BFP4])
@pytest.mark.parametrize("m,k,n", [(32, 64, 128), (32, 2048, 256), (32, 4096, 96)])
def test_gated_block_float_output(oracle, out_fmt, m, k, n):
    """Output dtype BFLOAT8_B / BFLOAT4_B of the gated launch (TILE layout): the words that packing its bf16 output gives
    (ttmi_typecast_tiles, itself pinned against the oracle's packer), stored directly and through the hand-over of partial
    sums, with a column group that is not full."""
    a_tiles = capi.tilize(bf16_dev(workloads.activations_bf16(m, k, seed=340)))
    gate_words, _ = pack_weights(oracle, workloads.weights_f32(k, n, seed=341), BFP4)
    up_words, _ = pack_weights(oracle, workloads.weights_f32(k, n, seed=342), BFP4)
    dense = capi.matmul_bfp_gated(a_tiles, capi.TILE, gate_words, up_words, BFP4, 1, 1, m, k, n, c_layout=capi.TILE)
    want = capi.typecast_tiles(dense, capi.BFLOAT16, out_fmt)
    got = capi.matmul_bfp_gated(a_tiles, capi.TILE, gate_words, up_words, BFP4, 1, 1, m, k, n, c_layout=capi.TILE, out_bfp=out_fmt)
    assert torch.equal(got, want)
    host = oracle.pack_fp32_vec_as_bfp_tiles(out_fmt, dense.float().cpu().numpy().reshape(-1), False)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), host)
