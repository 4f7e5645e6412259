"""The build-time assembly check of the streaming GEMM (tt-metal_amd/check_isa.py) on small hand-made listings:
it must accept a loop that takes loaded registers over with an inline move after its own wait, and reject a
compiler-generated copy of a register whose load is still in flight, also when the copy sits on a loop back edge."""
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "tt-metal_amd"))
import check_isa  # noqa: E402

HEAD = "_Z20matmul_stream_kernelILi7ELi0EEvN4ttmi9MatmulDevE:\n"
TAIL = "\ts_endpgm\n.Lfunc_end0:\n"


def asm(*lines):
    return "\t;;#ASMSTART\n" + "".join(f"\t{l}\n" for l in lines) + "\t;;#ASMEND\n"


def run(tmp_path, body):
    f = tmp_path / "k.s"
    f.write_text(HEAD + body + TAIL)
    return check_isa.check(str(f))


LOOP_OK = (
    asm("global_load_dwordx4 v[8:11], v[0:1], off")
    + ".LBB0_1:\n"
    + "\ts_waitcnt vmcnt(0) lgkmcnt(15)\n"      # stands for the kernel's own partial wait; see LOOP_PARTIAL below
    + asm("v_mov_b32 v20, v8", "v_mov_b32 v21, v9", "v_mov_b32 v22, v10", "v_mov_b32 v23, v11")
    + asm("global_load_dwordx4 v[8:11], v[0:1], off")
    + "\tv_add_u32_e32 v30, v20, v21\n"
    + "\ts_cbranch_scc1 .LBB0_1\n"
    + "\ts_waitcnt vmcnt(0)\n"
)


def test_clean_loop_passes(tmp_path):
    assert run(tmp_path, LOOP_OK) == 0


def test_partial_wait_and_inline_moves_release_the_registers(tmp_path):
    body = (
        asm("global_load_dwordx4 v[8:11], v[0:1], off", "global_load_dwordx4 v[12:15], v[0:1], off")
        + "\ts_waitcnt vmcnt(1)\n"
        + asm("v_mov_b32 v20, v8", "v_mov_b32 v21, v9", "v_mov_b32 v22, v10", "v_mov_b32 v23, v11")
        + "\tv_add_u32_e32 v8, v20, v21\n"        # v8..v11 are free again
        + "\ts_waitcnt vmcnt(0)\n"
        + "\tv_add_u32_e32 v12, v12, v13\n"
    )
    assert run(tmp_path, body) == 0


def test_compiler_copy_of_a_register_in_flight_is_reported(tmp_path, capsys):
    body = asm("global_load_dwordx4 v[8:11], v[0:1], off") + "\tv_mov_b64_e32 v[40:41], v[10:11]\n\ts_waitcnt vmcnt(0)\n"
    assert run(tmp_path, body) == 1
    assert "v_mov_b64_e32 v[40:41], v[10:11]" in capsys.readouterr().err


def test_flight_across_a_back_edge_is_followed(tmp_path):
    body = (
        ".LBB0_1:\n"
        + "\tv_add_u32_e32 v30, v8, v30\n"        # second trip: v8 has a load in flight from the first
        + asm("global_load_dwordx4 v[8:11], v[0:1], off")
        + "\ts_cbranch_scc1 .LBB0_1\n"
        + "\ts_waitcnt vmcnt(0)\n"
    )
    assert run(tmp_path, body) == 1


def test_load_in_flight_at_the_end_is_reported(tmp_path):
    assert run(tmp_path, asm("global_load_dwordx4 v[8:11], v[0:1], off")) == 1


def test_slot_loads_need_a_full_wait(tmp_path):
    body = (
        asm("global_load_dwordx4 v[24:27], v[0:1], off")
        + "\ts_waitcnt vmcnt(0)\n"
        + asm("global_load_dwordx4 v[8:11], v[0:1], off sc1")
        + asm("v_mov_b32 v20, v8")                 # an inline move does not end the flight of a slot load
        + "\tv_add_f32_e32 v12, v8, v9\n"
        + "\ts_waitcnt vmcnt(0)\n"
    )
    assert run(tmp_path, body) == 1


def test_a_listing_without_the_kernel_or_without_its_loads_fails(tmp_path):
    f = tmp_path / "none.s"
    f.write_text("_Z5otherv:\n\ts_endpgm\n.Lfunc_end0:\n")
    assert check_isa.check(str(f)) == 1
    assert run(tmp_path, "\tv_add_u32_e32 v1, v2, v3\n") == 1


def test_inline_lds_reads_are_in_flight_until_lgkmcnt_zero(tmp_path, capsys):
    ring = asm("global_load_dwordx4 v[8:11], v[0:1], off") + "\ts_waitcnt vmcnt(0)\n"   # the kernel must have ring loads
    good = ring + asm("ds_read2_b32 v[40:41], v5 offset0:0 offset1:4", "s_waitcnt lgkmcnt(0)") + "\tv_add_u32_e32 v42, v40, v41\n"
    assert run(tmp_path, good) == 0
    bad = ring + asm("ds_read2_b32 v[40:41], v5 offset0:0 offset1:4") + "\tv_mov_b32_e32 v50, v41\n" + asm("s_waitcnt lgkmcnt(0)")
    assert run(tmp_path, bad) == 1
    assert "v_mov_b32_e32 v50, v41" in capsys.readouterr().err
    # the compiler's own combined wait releases them as well
    also_good = ring + asm("ds_read_b64 v[40:41], v5 offset:32") + "\ts_waitcnt vmcnt(0) lgkmcnt(0)\n\tv_add_u32_e32 v42, v40, v41\n"
    assert run(tmp_path, also_good) == 0


# ---- the 384-row GEMM: ring registers are read by the MFMAs directly, behind the kernel's own partial wait -------------
TALL_HEAD = "_ZN4ttmi18matmul_tall_kernelILi7ELi0ELi12EEEvNS_7TileDevE:\n"


def run_tall(tmp_path, body):
    f = tmp_path / "t.s"
    f.write_text(TALL_HEAD + body + TAIL)
    return check_isa.check_ring_operands(str(f))


TALL_OK = (
    "\tv_mov_b32_e32 v34, 0\n\tv_mov_b32_e32 v35, v34\n"                    # zero initialisation before the first load
    + asm("global_load_dwordx4 v[34:37], v116, s[4:5]")
    + ".LBB0_1:\n"
    + "\ts_waitcnt vmcnt(2)\n\ts_barrier\n"
    + "\tv_mfma_f32_32x32x16_bf16 v[2:17], v[34:37], v[82:85], v[2:17]\n"
    + "\tv_mfma_f32_32x32x16_bf16 v[18:33], v[34:37], v[86:89], v[18:33]\n"
    + asm("global_load_dwordx4 v[34:37], v116, s[4:5]")
    + "\ts_cbranch_scc1 .LBB0_1\n"
    + "\ts_waitcnt vmcnt(0)\n"
)


def test_tall_kernel_ring_read_only_by_mfma_passes(tmp_path):
    assert run_tall(tmp_path, TALL_OK) == 0


def test_tall_kernel_copy_of_a_ring_register_in_flight_is_rejected(tmp_path):
    bad = TALL_OK.replace("\ts_cbranch_scc1 .LBB0_1\n", "\tv_mov_b32_e32 v90, v35\n\ts_cbranch_scc1 .LBB0_1\n")
    assert run_tall(tmp_path, bad) > 0


def test_tall_kernel_mfma_writing_a_ring_register_in_flight_is_rejected(tmp_path):
    bad = TALL_OK.replace("\ts_waitcnt vmcnt(2)\n", "\tv_mfma_f32_32x32x16_bf16 v[34:49], v[50:53], v[82:85], v[34:49]\n\ts_waitcnt vmcnt(2)\n")
    assert run_tall(tmp_path, bad) > 0


def test_tall_kernel_without_inline_loads_is_reported(tmp_path):
    assert run_tall(tmp_path, "\tv_mfma_f32_32x32x16_bf16 v[2:17], v[34:37], v[82:85], v[2:17]\n") > 0
