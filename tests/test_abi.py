"""The C-ABI library loads and exports every symbol include/ttmi.h declares (no compute, no GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ttmi.h")).read()
    return sorted(set(re.findall(r"TTMI_API[^;(]*?\b(ttmi_\w+)\s*\(", text)))


def test_header_symbols_are_exported():
    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libttmi.so not built in this checkout (python tt-metal_amd/build.py)")
    names = declared_symbols()
    assert len(names) >= 12
    assert sorted(capi.SYMBOLS) == names
    L = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(L, n), n


def test_the_product_library_has_no_test_hooks():
    """The ttmi_test_* entry points (forcing a kernel, dropping partial sums ...) exist in libttmi_test.so only."""
    import subprocess

    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH) or not os.path.exists(capi.LIB_TEST_PATH):
        pytest.skip("libraries not built")
    exported = lambda path: {line.split()[-1] for line in subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout.splitlines() if line.strip()}
    product, test = exported(capi.LIB_PATH), exported(capi.LIB_TEST_PATH)
    assert not [s for s in product if "ttmi_test" in s]
    assert {"ttmi_test_set_knob", "ttmi_test_kernel_choice", "ttmi_test_allocations"} <= test
    assert {s for s in product if s.startswith("ttmi_")} == {s for s in test if s.startswith("ttmi_") and not s.startswith("ttmi_test_")}


def test_size_helpers_need_no_gpu():
    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libttmi.so not built")
    L = capi.lib()
    # tt_backend_api_types.hpp:109-132
    assert [L.ttmi_tile_size(d) for d in (3, 4, 0, 1, 2, 6, 5)] == [1088, 576, 2048, 4096, 4096, 2048, 0]
    assert L.ttmi_tiled_size_bytes(3, 1, 1024, 1024) == 1114112
    assert L.ttmi_tiled_size_bytes(4, 1, 4096, 4096) == 9437184
    assert L.ttmi_tiled_size_bytes(3, 6, 7, 3) == 6 * 1088


def test_matmul_workspace_sizes_follow_the_decomposition():
    """What a caller has to bring for a GEMM of its own stream: 16 KB of partial-sum slots per computing workgroup of the
    128-column kernel (one band of rows), nothing when every output has a workgroup of its own, the expanded weights
    (2 bytes each) from 512 rows on."""
    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libttmi.so not built")
    ws = capi.lib().ttmi_matmul_bfp_workspace_bytes
    assert ws(1, 32, 4544, 18176, 3) == 142 * 3 * 16384        # 142 groups of 128 columns, 512 // 143 = 3 k ranges each
    assert ws(1, 32, 18176, 4544, 3) == 36 * 7 * 16384         # 36 groups (the last one half empty), 256 // 36 = 7
    assert ws(1, 32, 64, 4096, 3) == 0                         # 2 k-tiles: never shared
    assert ws(1, 64, 4544, 18176, 3) == 142 * 3 * 2 * 16384    # two bands per workgroup of the 128-column kernel: two slots each
    assert ws(1, 96, 4544, 18176, 3) == 0                      # three bands, 64-column kernel: 3 x 284 groups fill the chip
    assert ws(12, 384, 1024, 1024, 3) == 0                     # fused tiled kernels
    assert ws(1, 256, 4096, 4096, 3) == 128 * 4 * 2 * 16384    # too few blocks for the tiled kernels: streamed, 4 pairs of bands x 32 groups, 4 k ranges each (512 workgroups; those that only collect come on top), two slots per workgroup
    assert ws(1, 2048, 4096, 14336, 3) == 4096 * 14336 * 2     # expanded weights
    assert ws(0, 32, 64, 64, 3) == 0


def test_argument_validation_returns_errors_without_launching():
    from ttmi import capi

    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libttmi.so not built")
    L = capi.lib()
    assert L.ttmi_pack_fp32_vec_as_bfp_tiles(0, None, 1, 0, None, None) == 1
    assert b"BFLOAT8_B" in L.ttmi_last_error()
    assert L.ttmi_pack_fp32_vec_as_bfp_tiles(3, None, 1, 0, None, None) == 1
    assert L.ttmi_tilize(None, 3, 1, 32, 32, None, None) == 1
    one = ctypes.c_void_p(16)
    # K, N must be tile multiples; weight batch 1 or batch
    assert L.ttmi_matmul_bfp(one, 0, one, 3, 1, 1, 32, 33, 64, None, 0, one, 0, 0, None, 0, None) == 1
    assert b"multiples of 32" in L.ttmi_last_error()
    assert L.ttmi_matmul_bfp(one, 0, one, 3, 4, 2, 32, 32, 64, None, 0, one, 0, 0, None, 0, None) == 1
    assert L.ttmi_matmul_bfp(one, 1, one, 3, 1, 1, 7, 32, 64, None, 0, one, 0, 0, None, 0, None) == 1
    assert L.ttmi_matmul_bfp(one, 0, one, 2, 1, 1, 32, 32, 64, None, 0, one, 0, 0, None, 0, None) == 1
    # dense weight dtypes (BFLOAT16 = 0, FLOAT32 = 1) pass only through ttmi_matmul_bf16: every other matmul entry point would
    # decode them as packed tiles, so each refuses them before anything is launched
    for dense in (0, 1):
        assert L.ttmi_matmul_bfp(one, 0, one, dense, 1, 1, 32, 32, 64, None, 0, one, 0, 0, None, 0, None) == 1
        assert b"weight dtype" in L.ttmi_last_error()
        assert L.ttmi_matmul_bfp_static(one, 0, one, dense, 1, 1, 32, 32, 64, None, 0, one, 0, 0, None) == 1
        assert b"weight dtype" in L.ttmi_last_error()
        assert L.ttmi_matmul_bfp_gated(one, 0, one, one, dense, 1, 1, 32, 32, 64, None, 0, one, 0, 0, None, 0, None) == 1
        assert b"weight dtype" in L.ttmi_last_error()


def test_missing_library_fails_loudly(monkeypatch):
    from ttmi import capi

    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", "/nonexistent/libttmi.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        capi.lib()


# ---- host bookkeeping of the streaming GEMM kernels (no GPU) -------------------------------------------------------------
def _test_entries():
    from ttmi import capi

    if not os.path.exists(capi.LIB_TEST_PATH):
        pytest.skip("libttmi_test.so not built")
    L = capi._load(capi.LIB_TEST_PATH)          # the build with the ttmi_test_* entry points; the product library has none
    u32 = ctypes.c_uint32
    L.ttmi_test_stream_decomposition.restype = None
    L.ttmi_test_stream_decomposition.argtypes = [u32, u32, u32, u32, ctypes.c_int, ctypes.POINTER(u32)]
    L.ttmi_test_range_start.restype = u32
    L.ttmi_test_range_start.argtypes = [u32, u32, u32]
    L.ttmi_test_workgroup_of.restype = u32
    L.ttmi_test_workgroup_of.argtypes = [u32, u32, u32]
    L.ttmi_test_scratch_grown_size.restype = ctypes.c_size_t
    L.ttmi_test_scratch_grown_size.argtypes = [ctypes.c_size_t, ctypes.c_size_t]
    return L


SHAPES = [(1, 32, 4544, 18176), (1, 32, 18176, 4544), (1, 32, 4096, 6144), (1, 32, 4096, 4096), (1, 32, 14336, 4096),
          (1, 32, 4096, 14336), (3, 24, 768, 160), (2, 40, 1024, 288), (1, 8, 32, 32), (1, 32, 64, 4096), (5, 100, 96, 2080)]


def test_kernel_choice_by_shape():
    """Which kernel a GEMM goes to: one band streams in 128-column units, unless its 64-column groups are one workgroup per CU
    (200 to 256 of them) of at most 192 KiB of BFP4_B weights each and the output is not block-float — then the 64-column kernel
    takes it with one workgroup per group and nothing shared; two and four bands in the two-band form, three in 64-column
    units when the GEMM has more columns than rows of weights; from 128 rows on tiled (up to 511 rows) or expanded where the output has blocks enough to fill the chip, else
    streamed in the two-band form."""
    from ttmi import capi

    L = _test_entries()
    u32 = ctypes.c_uint32
    L.ttmi_test_kernel_choice.restype = ctypes.c_int
    L.ttmi_test_kernel_choice.argtypes = [u32, u32, u32, u32, ctypes.c_int, ctypes.c_int]
    STREAM, WIDE, TILE, EXPANDED = 1, 2, 3, 4
    B8, B4, BF16 = capi.BFLOAT8_B, capi.BFLOAT4_B, capi.BFLOAT16
    cases = [((1, 32, 4544, 18176, B8, BF16), WIDE), ((1, 32, 18176, 4544, B8, BF16), WIDE), ((1, 32, 4096, 4096, B8, BF16), WIDE),
             ((1, 32, 4096, 14336, B4, BF16), STREAM), ((1, 32, 4096, 14336, B4, B8), WIDE), ((1, 32, 4096, 14336, B8, BF16), WIDE),
             ((1, 32, 4096, 16384, B4, BF16), STREAM), ((1, 32, 4096, 16448, B4, BF16), WIDE), ((1, 32, 4096, 12736, B4, BF16), WIDE),
             ((1, 32, 14336, 4096, B4, BF16), WIDE), ((2, 20, 1024, 7168, B8, BF16), WIDE), ((2, 20, 1024, 7168, B4, BF16), STREAM), ((1, 32, 8192, 14336, B4, BF16), WIDE), ((1, 64, 4096, 14336, B4, BF16), WIDE),
             ((1, 96, 4096, 4096, B8, BF16), WIDE), ((1, 96, 4096, 14336, B4, BF16), STREAM), ((1, 96, 14336, 4096, B4, BF16), WIDE), ((1, 2048, 4096, 14336, B8, BF16), EXPANDED),
             # from 128 rows on: blocks of the output where there are enough of them to fill the chip, else the weights are streamed
             ((1, 128, 4096, 4096, B8, BF16), WIDE), ((1, 256, 4096, 14336, B8, BF16), WIDE), ((1, 128, 14336, 4096, B8, BF16), WIDE),
             ((12, 384, 1024, 1024, B8, BF16), TILE), ((1, 256, 512, 32768, B8, BF16), TILE), ((4, 256, 1024, 8192, B8, BF16), TILE),
             ((1, 1024, 4096, 14336, B8, BF16), EXPANDED), ((1, 512, 4096, 1024, B8, BF16), WIDE)]
    for args, want in cases:
        assert L.ttmi_test_kernel_choice(*args) == want, args
    # the public form of the same answer (for reading profiler traces): kernel, k ranges per output, grid with and without
    # the output groups dealt out to 8 XCDs
    L.ttmi_test_stream_decomposition.restype = None
    L.ttmi_test_stream_decomposition.argtypes = [u32, u32, u32, u32, ctypes.c_int, ctypes.POINTER(u32)]
    P = capi.lib()
    for args, want in cases:
        plan, dec = (u32 * 4)(), (u32 * 4)()
        P.ttmi_matmul_bfp_plan(*args[:4], BF16, args[4], args[5], plan)
        assert plan[0] == want, args
        if want in (STREAM, WIDE):
            L.ttmi_test_stream_decomposition(*args[:4], int(want == WIDE), dec)
            groups, split, workgroups = dec[0], dec[2], dec[3]
            assert plan[1] == split
            assert plan[2] == (workgroups + (split if want == WIDE and split > 1 else 0))
            dealt = want == WIDE and split > 1 and ((groups + 7) // 8) * 8 * 32 <= groups * 33
            assert plan[3] == (8 * ((groups + 7) // 8 + 1) * split if dealt else plan[2]), args
        else:
            assert list(plan[1:]) == [0, 0, 0]
    plan = (u32 * 4)()
    P.ttmi_matmul_bfp_plan(1, 32, 4544, 18176, BF16, B8, BF16, plan)
    assert list(plan) == [WIDE, 3, 429, 456]                                # Falcon h_to_4h: 142 groups x 3, + 3 collectors | 8 x 19 x 3
    P.ttmi_matmul_bfp_plan(1, 32, 4096, 14336, B8, B4, BF16, plan)          # block-float activations keep the 64-column kernel out
    assert plan[0] == WIDE
    # the one-round form: one workgroup per group, no partial sums, no workspace
    out = (u32 * 4)()
    L.ttmi_test_stream_decomposition(1, 32, 4096, 14336, 0, out)
    assert [int(x) for x in out] == [224, 128, 1, 224]
    # the workspace query covers the 128-column kernel, which the same shape takes with a block-float output
    L.ttmi_test_stream_decomposition(1, 32, 4096, 14336, 1, out)
    assert L.ttmi_matmul_bfp_workspace_bytes(1, 32, 4096, 14336, B4) == int(out[3]) * 16384


@pytest.mark.parametrize("wide", [0, 1])
@pytest.mark.parametrize("shape", SHAPES)
def test_every_unit_has_exactly_one_workgroup_and_collectors_come_last(shape, wide):
    """The two functions the kernels cut the work with, on the decompositions the host chooses: the k ranges of an output
    tile it without gap or overlap, workgroup_of inverts range_start, and whoever collects an output has a higher index
    than every workgroup that contributes to it — the collectors wait for lower indices only.  (That lower indices are
    dispatched first and therefore finish without waiting for anybody is an assumption about the hardware's dispatcher,
    not a guarantee of the programming model; the bounded wait and the error word cover the case that it fails.)"""
    L = _test_entries()
    L.ttmi_test_wide_workgroup_number.restype = ctypes.c_uint32
    L.ttmi_test_wide_workgroup_number.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
    out = (ctypes.c_uint32 * 4)()
    L.ttmi_test_stream_decomposition(*shape, wide, out)
    groups, kt, split, workgroups = (int(x) for x in out)
    batch, m, k, n = shape
    bands = -(-m // 32)
    band_sets = -(-bands // 2) if wide and m > 32 else bands        # the 128-column kernel takes two bands per workgroup above 32 rows
    assert kt == k // 32 and groups == batch * band_sets * -(-(n // 32) // (4 if wide else 2))
    assert split >= 1 and workgroups == groups * split
    assert split == 1 or kt // split >= 2                     # every wavefront of a shared output keeps work to do
    starts = [L.ttmi_test_range_start(kt, split, i) for i in range(min(workgroups, 600) + 1)]
    for i in range(len(starts) - 1):
        og, part = divmod(i, split)
        assert og * kt <= starts[i] < starts[i + 1] <= (og + 1) * kt          # non-empty, inside its own output
        if part == 0:
            assert starts[i] == og * kt                                         # the first range starts the output
        for unit in {starts[i], starts[i + 1] - 1, (starts[i] + starts[i + 1]) // 2}:
            assert L.ttmi_test_workgroup_of(kt, split, unit) == i
    if split > 1:
        # wide kernel: the `split` workgroups of output g + 1 (after the last output: `split` extra workgroups) collect
        # output g; 64-column kernel: the contributor with the highest index collects
        for g in range(min(groups, 50)):
            contributors = range(g * split, (g + 1) * split)
            collectors = range((g + 1) * split, (g + 2) * split) if wide else [contributors[-1]]
            assert min(collectors) >= max(contributors) and (not wide or min(collectors) > max(contributors))
    if split > 1 and wide:
        # The same kernel with the output groups dealt out to 8 XCDs (hardware index b -> XCD b % 8 + c, number b / 8 there):
        # the launch has one more round of `split` workgroups per XCD; every (group, part) has exactly one workgroup, all
        # contributors and collectors of a group share b % 8, i.e. an XCD, and the collectors (the group 8 further on) still
        # have the higher hardware indices.
        grid = 8 * (-(-groups // 8) + 1) * split
        number = [L.ttmi_test_wide_workgroup_number(b, split) for b in range(grid)]
        assert sorted(number) == list(range(grid))
        where = {n: b for b, n in enumerate(number)}
        for g in range(min(groups, 60)):
            contributors = [where[g * split + part] for part in range(split)]
            collectors = [where[(g + 8) * split + part] for part in range(split)]
            assert len({b % 8 for b in contributors + collectors}) == 1
            assert min(collectors) > max(contributors)


def test_division_by_host_known_divisors():
    """The kernels divide by numbers the host knows (k ranges per output, groups per band) with a multiplication and a shift;
    exact for every dividend below 2^31 — checked at the edges of every quotient for a spread of divisors."""
    L = _test_entries()
    L.ttmi_test_fast_div.restype = ctypes.c_uint32
    L.ttmi_test_fast_div.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
    import random
    rng = random.Random(5)
    divisors = list(range(1, 70)) + [71, 112, 127, 128, 129, 142, 255, 256, 257, 568, 1000, 4095, 4096, 4097, 65535, 65536, 1 << 20, (1 << 26) - 1, (1 << 30) + 1]
    for d in divisors:
        top = (1 << 31) - 1
        samples = {0, 1, d - 1, d, d + 1, top, top - 1, top // d * d, max(top // d * d - 1, 0)}
        for _ in range(40):
            q = rng.randrange(0, top // d + 1)
            samples.update({min(q * d, top), min(q * d + d - 1, top), max(q * d - 1, 0)})
        for n in samples:
            assert L.ttmi_test_fast_div(n, d) == n // d, (n, d)


def test_library_scratch_grows_geometrically_and_is_never_shrunk():
    """A buffer that is too small is replaced by one of at least twice its size (the old one is retired, not freed: a
    kernel of another host thread may still be about to use it), so the retired buffers of a stream add up to less than
    the live one; sizes are multiples of 256 bytes."""
    L = _test_entries()
    grown = L.ttmi_test_scratch_grown_size
    assert grown(0, 1) == 256 and grown(0, 16384) == 16384 and grown(4096, 100) == 4096
    assert grown(16384, 16385) == 32768 and grown(16384, 100000) == 100096
    have, retired = 0, 0
    for need in (1000, 5000, 5001, 70000, 70001, 300000):
        new = grown(have, need)
        assert new >= need and new % 256 == 0
        if new != have:
            retired += have
            assert have == 0 or new >= 2 * have
            have = new
    assert retired < have


def test_test_knobs_are_validated_and_cleared(knobs):
    from ttmi import capi

    L = _test_entries()
    ws = L.ttmi_matmul_bfp_workspace_bytes
    assert ws(1, 32, 4544, 18176, 3) == 142 * 3 * 16384
    knobs("workgroups", 256)
    assert ws(1, 32, 4544, 18176, 3) == 0                       # 256 // 143 = 1 k range per output: nothing is shared
    knobs("kernel", "expanded")
    assert ws(1, 32, 64, 64, 3) == 2 * 1 * 4096                 # forced onto the expanding kernel: one 64-column group, two k tiles
    L.ttmi_test_set_knob.restype = ctypes.c_int
    assert L.ttmi_test_set_knob(99, 0, 1) == 1 and b"unknown test knob" in L.ttmi_last_error()


@pytest.mark.parametrize("bits,tile_bytes", [(7, 1088), (3, 576)])
def test_lds_stage_of_the_wide_kernel(bits, tile_bytes):
    """The LDS stage of the 128-column GEMM kernel, from the addresses its own code computes (test entry point): every
    mantissa word and exponent byte a lane reads is the one of its tile, face, k row and column quad; the 64 lanes of every
    pass of a ds_read2_b32 and of the exponent read fall into 64 different banks of 4 bytes, and the 32 lanes of either half
    into 32 different banks when only address bits 2..6 choose the bank; and every four neighbouring
    lanes of a load fetch one aligned 64-byte piece of memory (what the vector memory pipe coalesces)."""
    from ttmi import capi

    L = _test_entries()
    L.ttmi_test_wide_layout.restype = None
    L.ttmi_test_wide_layout.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_uint32)]
    lanes = []
    for lane in range(64):
        out = (ctypes.c_uint32 * 16)()
        L.ttmi_test_wide_layout(bits, lane, out)
        lanes.append([int(x) for x in out])
    loads, load_stride, unit_bytes, slab_bytes, row_step = lanes[0][:5]
    pair_offsets = lanes[0][5:9]
    row_bytes, face_bytes = (16, 256) if bits == 7 else (8, 128)
    assert row_step == row_bytes
    stage = {}                                               # LDS byte of the stage -> byte of the unit's 4 tiles in memory
    for l in range(loads):
        for lane in range(64):
            chunk = lanes[lane][11 + l]
            assert chunk < 4 * tile_bytes // 16
            for b in range(16):
                at = l * load_stride + lane * 16 + b
                assert at < unit_bytes
                stage[at] = chunk * 16 + b
        for quad in range(16):
            assert len({lanes[quad * 4 + j][11 + l] // 4 for j in range(4)}) == 1
    for s in range(2):
        exp_banks = set()
        for lane in range(64):
            c32, kh = lane & 31, lane >> 5
            t, fc = c32 >> 3, (c32 >> 2) & 1
            at = lanes[lane][9] + 32 * s
            assert [stage[at + b] for b in range(8)] == [t * tile_bytes + (2 * s + fc) * 16 + kh * 8 + b for b in range(8)]
            exp_banks.update({(at // 4) % 64, (at // 4 + 1) % 64})
        assert len(exp_banks) == 32                           # 16 different addresses of 8 bytes, the four lanes of a column quad share one
        for i in range(4):
            for second in range(2):
                banks = set()
                for lane in range(64):
                    c32, kh = lane & 31, lane >> 5
                    t, fc, q = c32 >> 3, (c32 >> 2) & 1, c32 & 3
                    word = q if bits == 7 else q >> 1
                    at = lanes[lane][10] + s * slab_bytes + pair_offsets[i] + second * row_step
                    want = t * tile_bytes + 64 + (2 * s + fc) * face_bytes + (8 * kh + 2 * i + second) * row_bytes + word * 4
                    assert [stage[at + b] for b in range(4)] == [want + b for b in range(4)]
                    banks.add(((at // 4) % 64, at))
                assert len({b for b, _ in banks}) == len({a for _, a in banks})     # different addresses, different banks
                assert len({a for _, a in banks}) == (64 if bits == 7 else 32)         # BFP4: two lanes share a word
                # the same for half a wavefront at a time on 32 banks (what the bank-conflict counter of the hardware fits)
                for half in range(2):
                    addresses = set()
                    for lane in range(32 * half, 32 * half + 32):
                        addresses.add(lanes[lane][10] + s * slab_bytes + pair_offsets[i] + second * row_step)
                    assert len({(a // 4) % 32 for a in addresses}) == len(addresses)
