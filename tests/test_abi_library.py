"""CPU-only checks of the C ABI library: it loads without a GPU, exports every symbol declared in
include/mi355x_rownorm.h, validates arguments before touching the device, and plans launches the
way the header documents.  No kernel is launched here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355x_rownorm.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355x_\w+)\s*\(", text)))


def test_header_and_python_binding_agree(cabi):
    assert declared_functions() == sorted(cabi.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol(cabi):
    lib = cabi.lib()
    for name in declared_functions():
        assert getattr(lib, name) is not None, name
    assert lib.mi355x_rownorm_abi_version() == 1


def test_error_strings(cabi):
    assert cabi.error_string(0) == "success"
    for code in (-1, -2, -3, -4, -5, -6):
        assert "mi355x_rownorm" in cabi.error_string(code)
    assert cabi.error_string(-99).startswith("mi355x_rownorm: unknown")


def test_argument_validation_happens_before_any_launch(cabi):
    L = cabi.lib()
    null = None
    # unknown dtype code, unsupported dtype pair
    assert L.mi355x_layer_norm_fwd(null, null, null, null, null, null, 4, 8, 1e-5, 7, 0, null) == -1
    assert L.mi355x_rms_norm_fwd(null, null, null, null, 4, 8, 1e-5, cabi.F32, cabi.BF16, null) == -1
    assert L.mi355x_softmax_fwd(null, null, 4, 8, cabi.BF16, cabi.F32, 0, null) == -1  # only f16->f32
    assert L.mi355x_softmax_bwd(null, null, null, 4, 8, cabi.F32, cabi.BF16, 0, null) == -1
    # negative sizes / oversize rows
    assert L.mi355x_layer_norm_fwd(null, null, null, null, null, null, -1, 8, 1e-5, 0, 0, null) == -2
    assert L.mi355x_softmax_fwd(null, null, 4, (1 << 30) + 1, 0, 0, 0, null) == -2
    # empty problems are a successful no-op even with null pointers (M == 0 or N == 0)
    assert L.mi355x_layer_norm_fwd(null, null, null, null, null, null, 0, 8, 1e-5, 0, 0, null) == 0
    assert L.mi355x_rms_norm_bwd(null, null, null, null, null, null, null, 0, 5, 0, 0, 0, null) == 0
    assert L.mi355x_softmax_bwd(null, null, null, 0, 8, 0, 0, 1, null) == 0
    # required pointers
    assert L.mi355x_layer_norm_fwd(null, null, null, null, null, null, 4, 8, 1e-5, 0, 0, null) == -3
    assert L.mi355x_softmax_fwd(null, null, 4, 8, 0, 0, 0, null) == -3
    # backward with column sums wanted but no workspace
    one = ctypes.c_void_p(256)  # never dereferenced: the call is rejected before launching
    assert L.mi355x_layer_norm_bwd(one, one, one, one, one, one, one, one, null, 0, 4, 8, 0, 0,
                                   null) == -4
    assert L.mi355x_rms_norm_bwd(one, one, one, one, one, one, null, 0, 4, 8, 0, 0, null) == -4
    # nothing requested: no-op
    assert L.mi355x_rms_norm_bwd(one, one, one, one, null, null, null, 0, 4, 8, 0, 0, null) == 0


def test_mask_row_mapping_is_bounds_checked_before_any_launch(cabi):
    L = cabi.lib()
    one, null = ctypes.c_void_p(256), None  # never dereferenced: every call here is rejected
    fwd = lambda rows, N, mrows, div, stride, mod, mask=one: L.mi355x_masked_softmax_fwd(
        one, mask, one, rows, N, mrows, div, stride, mod, cabi.F32, null)
    bwd = lambda rows, N, mrows, div, stride, mod, mask=one: L.mi355x_masked_softmax_bwd(
        one, one, mask, one, rows, N, mrows, div, stride, mod, cabi.F32, null)
    for call in (fwd, bwd):
        assert call(8, 16, 8, 1, 1, 1, mask=null) == -3          # mask missing
        assert call(0, 16, 0, 1, 1, 1, mask=null) == 0           # empty problem: no-op
        assert call(8, 16, 7, 1, 1, 1) == -2                     # full mask one row short
        assert call(8, 16, 8, 0, 1, 1) == -2                     # div must be positive
        assert call(8, 16, 8, 1, -1, 1) == -2                    # negative stride
        assert call(8, 16, 8, 1, 1, 0) == -2                     # mod must be positive
        assert call(2 * 3 * 4, 4, 1, 12, 1, 1) == -2             # [B, T] mask with B = 2 given 1 row
        assert call(2 * 3 * 4, 4, 3, 1, 0, 4) == -2              # [T, T] mask with T = 4 given 3 rows
        assert call(2 * 3 * 4, 4, 7, 12, 4, 4) == -2             # [B, 1, T, T] needs B*T = 8 rows
        assert call(1 << 31, 4, 1 << 31, 1, 1, 1) == -2          # masked calls stop at 2^31 rows
    # dtype pairs: the masked entry points take one dtype for everything
    assert L.mi355x_masked_softmax_fwd(one, one, one, 8, 16, 8, 1, 1, 1, 9, null) == -1
    assert L.mi355x_safe_softmax_fwd(null, null, 4, 8, cabi.BF16, cabi.F32, null) == -1
    assert L.mi355x_safe_softmax_fwd(null, null, 4, 8, cabi.F16, cabi.F32, null) == -3
    assert L.mi355x_safe_softmax_fwd(null, null, 0, 8, cabi.F16, cabi.F32, null) == 0


def test_mask_row_map_helper(cabi):
    assert cabi.mask_row_map((2, 3, 4, 4), (2, 3, 4, 4)) == (24, 1, 1, 1)
    assert cabi.mask_row_map((2, 3, 4, 4), (2, 4)) == (2, 12, 1, 1)
    assert cabi.mask_row_map((2, 3, 4, 4), (4, 4)) == (4, 1, 0, 4)
    assert cabi.mask_row_map((2, 3, 4, 4), (2, 1, 4, 4)) == (8, 12, 4, 4)
    with pytest.raises(RuntimeError, match="does not fit"):
        cabi.mask_row_map((2, 3, 4, 4), (3, 4))
    # brute force: the mapping names the same mask row as numpy broadcasting does
    import numpy as np
    B, H, T = 2, 3, 4
    for mshape, view in (((B, T), (B, 1, 1, T)), ((T, T), (1, 1, T, T)), ((B, 1, T, T),) * 2,
                         ((B, H, T, T),) * 2):
        mrows, div, stride, mod = cabi.mask_row_map((B, H, T, T), mshape)
        ids = np.arange(mrows)[:, None].repeat(T, 1).reshape(mshape)       # mask row id per element
        full = np.broadcast_to(ids.reshape(view), (B, H, T, T)).reshape(-1, T)[:, 0]
        mapped = [(r // div) * stride + r % mod for r in range(B * H * T)]
        assert mapped == list(full), mshape


def test_workspace_size_follows_the_plan(cabi):
    L = cabi.lib()
    # The query covers every call of that shape: with or without dX, with or without a residual
    # gradient.  Those may take different layouts (a call that writes dX takes the exact two-pack
    # layout on one workgroup a compute unit, one that only sums columns the general kernel on
    # two), so the answer is at least what the reported plan needs and at most the largest grid.
    p = cabi.plan(cabi.OP_RMS_NORM_BWD, 16384, 4096, cabi.BF16, cabi.BF16)
    assert p["partial_rows"] == p["grid_blocks"] > 0
    nws = L.mi355x_rms_norm_bwd_workspace_bytes(16384, 4096, cabi.BF16, cabi.BF16, 1)
    assert p["partial_rows"] * 4096 * 4 <= nws <= 512 * 4096 * 4
    assert L.mi355x_rms_norm_bwd_workspace_bytes(16384, 4096, cabi.BF16, cabi.BF16, 0) == 0
    p = cabi.plan(cabi.OP_LAYER_NORM_BWD, 16384, 8192, cabi.BF16, cabi.F32)
    nws = L.mi355x_layer_norm_bwd_workspace_bytes(16384, 8192, cabi.BF16, cabi.F32, 1, 1)
    assert 2 * p["partial_rows"] * 8192 * 4 <= nws <= 2 * 512 * 8192 * 4
    # a shape with one layout for all of them: the answer is exactly the plan's partial rows
    p = cabi.plan(cabi.OP_LAYER_NORM_BWD, 16384, 8192, cabi.F32, cabi.F32)
    assert L.mi355x_layer_norm_bwd_workspace_bytes(16384, 8192, cabi.F32, cabi.F32, 1, 1) == \
        2 * p["partial_rows"] * 8192 * 4
    assert L.mi355x_layer_norm_bwd_workspace_bytes(16384, 8192, cabi.BF16, cabi.F32, 0, 0) == 0
    assert L.mi355x_layer_norm_bwd_workspace_bytes(0, 8192, cabi.BF16, cabi.F32, 1, 1) == 0


@pytest.mark.parametrize("op", range(6))
@pytest.mark.parametrize("dt", [0, 1, 2])
def test_plan_invariants(cabi, op, dt):
    esize = 4 if dt == 0 else 2
    E = 16 // esize
    for N in (1, 7, 8, 64, 127, 1000, 1024, 2048, 4096, 4097, 5120, 8192, 16384, 40000, 1 << 20):
        for M in (1, 3, 1000, 1 << 20):
            p = cabi.plan(op, M, N, dt, dt)
            assert p["grid_blocks"] >= 1
            if op in (cabi.OP_SOFTMAX_FWD, cabi.OP_SOFTMAX_BWD) and p["row_chunks"] > 0:
                # few, very long softmax rows of whole packs: a team of `row_chunks` workgroups
                # of 512 threads holds a row (16 packs a lane at most, the backward 8 of each
                # tensor), no more teams than rows
                team = p["row_chunks"]
                assert N % E == 0 and N // E >= 4096 and 2 * M <= 256, (M, N, p)
                assert team >= 2 and p["grid_blocks"] % team == 0 and p["grid_blocks"] <= 512
                assert 1 <= p["grid_blocks"] // team <= M
                assert team * 512 * (16 if op == cabi.OP_SOFTMAX_FWD else 8) * E >= N
            elif p["resident"]:
                G, V = p["lanes_per_row"], p["packs_per_lane"]
                # a power of two, or (exact two-pack layouts of the 16-bit norm backward) a
                # whole number of wavefronts
                assert 8 <= G <= 1024 and (G & (G - 1) == 0 or G % 64 == 0) and V >= 1
                assert G * V * E >= N, "row must fit the lanes' registers"
                assert p["block_threads"] % G == 0 and p["block_threads"] <= 1024
                assert p["rows_per_block"] == p["block_threads"] // G
                assert p["grid_blocks"] <= (M + p["rows_per_block"] - 1) // p["rows_per_block"]
            elif (op in (cabi.OP_LAYER_NORM_FWD, cabi.OP_RMS_NORM_FWD) and N % E == 0 and
                  p["row_chunks"] >= 2 and p["block_threads"] == 512 and
                  p["packs_per_lane"] == 10):
                # many forward rows of whole packs too long for eight teams at a time: a team of
                # `row_chunks` workgroups a row, ten packs a lane, one workgroup a compute unit,
                # three rows in flight; from 16 rounds on
                team = p["row_chunks"]
                assert p["rows_per_block"] == 1
                assert team == (N // E + 5119) // 5120 and p["grid_blocks"] <= 256
                teams = p["grid_blocks"] // team
                assert p["grid_blocks"] % team == 0 and 1 <= teams <= M
                assert M >= 16 * teams and 5 * (N // E) >= 4 * team * 5120
            elif (op in (cabi.OP_LAYER_NORM_FWD, cabi.OP_RMS_NORM_FWD) and N % E == 0 and
                  p["grid_blocks"] > M):
                # rows of whole packs beyond one workgroup's registers, 8 teams or more: a team
                # of `row_chunks` workgroups holds a row, at most one workgroup a compute unit,
                # no more teams than rows, every workgroup with at most 16 packs a lane
                team = p["row_chunks"]
                assert p["rows_per_block"] == 1 and team >= 1 and p["grid_blocks"] % team == 0
                assert p["grid_blocks"] <= 512 and 8 <= p["grid_blocks"] // team <= M
                assert team * 512 * 16 * E >= N
            elif (op in (cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_BWD) and N % E == 0 and
                  p["row_chunks"] >= 2 and p["block_threads"] == 512 and p["packs_per_lane"] == 2):
                # backward rows of whole packs beyond one workgroup's registers: a team of
                # `row_chunks` workgroups holds four rows at a time, two strides of 512 packs a
                # workgroup, one workgroup a compute unit, no more teams than groups of four
                # rows, one partial row a team
                team = p["row_chunks"]
                assert team == (N // E + 1023) // 1024 and p["grid_blocks"] <= 256
                assert p["grid_blocks"] % team == 0 and 1 <= p["grid_blocks"] // team <= (M + 3) // 4
                assert p["partial_rows"] >= p["grid_blocks"] // team
                # from the second round on (a LayerNorm on teams of more than 64: the fourth)
                groups, teams = (M + 3) // 4, p["grid_blocks"] // team
                if op == cabi.OP_LAYER_NORM_BWD and team > 64:
                    assert groups >= 4 * teams
                else:
                    assert groups > teams
            else:
                assert p["rows_per_block"] == 1 and p["grid_blocks"] <= M
            if op in (cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_BWD):
                assert p["partial_rows"] >= 1
            else:
                assert p["partial_rows"] == 0


def test_plan_query_for_tensors_off_a_cache_line(cabi):
    """The norm forwards and the softmax ops look at their pointers: rows of at most 64 packs in
    tensors off a 128-byte line take one pack a lane.  mi355x_rownorm_plan_at reports that layout;
    the norm backward takes it everywhere."""
    for op in (cabi.OP_LAYER_NORM_FWD, cabi.OP_RMS_NORM_FWD, cabi.OP_SOFTMAX_FWD,
               cabi.OP_SOFTMAX_BWD):
        for dt, E in ((cabi.F32, 4), (cabi.F16, 8)):
            for packs in (9, 16, 33, 64):
                on = cabi.plan(op, 4096, packs * E, dt, dt)
                off = cabi.plan(op, 4096, packs * E, dt, dt, off_line=True)
                assert on["packs_per_lane"] > 1, (op, dt, packs, on)
                assert off["packs_per_lane"] == 1 and off["lanes_per_row"] >= packs, (op, off)
            # longer rows do not change
            assert cabi.plan(op, 4096, 65 * E * 2, dt, dt) == cabi.plan(op, 4096, 65 * E * 2, dt, dt,
                                                                        off_line=True)
    for op in (cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_BWD):
        assert cabi.plan(op, 4096, 256, cabi.F32, cabi.F32) == \
            cabi.plan(op, 4096, 256, cabi.F32, cabi.F32, off_line=True)
        assert cabi.plan(op, 4096, 256, cabi.F32, cabi.F32)["packs_per_lane"] == 1


def test_override_fields_are_range_checked(cabi):
    L = cabi.lib()
    assert L.mi355x_rownorm_set_override(cabi.OP_SOFTMAX_FWD, 70000, 0, 0, 0) == -5
    assert L.mi355x_rownorm_set_override(cabi.OP_SOFTMAX_FWD, 0, -1, 0, 0) == -5
    assert L.mi355x_rownorm_set_override(cabi.OP_SOFTMAX_FWD, -2, 0, 0, 0) == -5
    assert L.mi355x_rownorm_set_override(99, 0, 0, 0, 0) == -2
    # a forced variant round-trips through the packed word, the multi-pass marker (-1) included
    cabi.set_override(cabi.OP_LAYER_NORM_FWD, -1, 5)
    p = cabi.plan(cabi.OP_LAYER_NORM_FWD, 4, 300000, cabi.F32, cabi.F32)
    assert p["resident"] == 0 and p["row_chunks"] == 5, p
    cabi.set_override(cabi.OP_LAYER_NORM_FWD, 512, 4, 512, 3)
    p = cabi.plan(cabi.OP_LAYER_NORM_FWD, 16384, 16384, cabi.BF16, cabi.BF16)
    assert (p["lanes_per_row"], p["packs_per_lane"], p["block_threads"]) == (512, 4, 512), p
    assert p["grid_blocks"] == 3 * 256
    cabi.clear_overrides()


def test_plan_picks_resident_kernels_for_the_llama_shapes(cabi):
    for op, M, N, dt in ((cabi.OP_LAYER_NORM_FWD, 4096, 1024, cabi.F32),
                         (cabi.OP_RMS_NORM_FWD, 16384, 4096, cabi.BF16),
                         (cabi.OP_RMS_NORM_BWD, 16384, 4096, cabi.BF16),
                         (cabi.OP_SOFTMAX_FWD, 262144, 2048, cabi.BF16),
                         (cabi.OP_SOFTMAX_BWD, 262144, 2048, cabi.BF16),
                         (cabi.OP_LAYER_NORM_FWD, 16384, 8192, cabi.BF16),
                         (cabi.OP_LAYER_NORM_BWD, 16384, 8192, cabi.BF16),
                         (cabi.OP_LAYER_NORM_BWD, 8192, 16384, cabi.F32)):
        assert cabi.plan(op, M, N, dt, dt)["resident"] == 1, (op, M, N, dt)
    # rows far beyond the register file stream through the multi-pass kernels
    assert cabi.plan(cabi.OP_SOFTMAX_FWD, 4, 1 << 20, cabi.F32, cabi.F32)["resident"] == 0


def test_plan_layouts_for_hidden_sizes_that_are_not_powers_of_two(cabi):
    """(lanes per row, packs per lane) of the measured exceptions to the power-of-two rule."""
    def lay(op, N, dt, wdt=None):
        p = cabi.plan(op, 16384, N, dt, dt if wdt is None else wdt)
        assert p["resident"] == 1
        return p["lanes_per_row"], p["packs_per_lane"]
    BF, F32 = cabi.BF16, cabi.F32
    LF, LB, RF, RB = (cabi.OP_LAYER_NORM_FWD, cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_FWD,
                      cabi.OP_RMS_NORM_BWD)
    # powers of two keep the rule: 2 packs (16-bit) / 4 packs (fp32) a lane
    assert lay(RF, 4096, BF) == (256, 2) and lay(RB, 4096, BF) == (256, 2)
    assert lay(LF, 8192, BF, F32) == (512, 2) and lay(LB, 8192, BF, F32) == (512, 2)
    assert lay(LF, 1024, F32) == (64, 4)
    # rows that fill at most 3/4 of the slots: three packs on fewer lanes (forward)
    for N, want in ((1536, (64, 3)), (3072, (128, 3)), (5120, (256, 3)), (6144, (256, 3))):
        if N != 5120:  # (the norm forward at 5120 takes an exact layout, below)
            assert lay(LF, N, BF) == want and lay(RF, N, BF) == want
        assert lay(cabi.OP_SOFTMAX_FWD, N, BF) == want
    # 16-bit forward rows of 4096 and 5120 elements: exact two-pack layouts on 256 / 320 lanes,
    # two 512-thread / three 320-thread resident workgroups a compute unit; an odd row count on
    # two row slots a workgroup, and the fused add, keep the general kernel
    for op in (LF, RF):
        p = cabi.plan(op, 16384, 4096, BF, BF)
        assert (p["lanes_per_row"], p["packs_per_lane"], p["block_threads"], p["grid_blocks"]) == (256, 2, 512, 512)
        p = cabi.plan(op, 16384, 5120, BF, F32)
        assert (p["lanes_per_row"], p["packs_per_lane"], p["block_threads"], p["grid_blocks"]) == (320, 2, 320, 768)
        p = cabi.plan(op, 16383, 4096, BF, BF)
        assert (p["lanes_per_row"], p["block_threads"]) == (256, 256)
    assert lay(LF, 7168, BF) == (512, 2)                       # fills 7/8: the rule stands
    # the 16-bit backward from 513 packs: three packs a lane, or an exact layout of six wavefronts
    assert lay(LB, 6160, BF) == (256, 4) or lay(LB, 6160, BF) == (512, 2)
    assert lay(LB, 5632, BF) == (256, 3) and lay(RB, 5632, BF) == (256, 3)
    assert lay(LB, 6144, BF) == (384, 2) and lay(RB, 6144, BF) == (384, 2)
    # 16-bit backward rows that are two packs on a whole number of wavefronts, where that
    # measured faster: the exact layouts (320 lanes for 5120, 448 for 7168, 1024 for the
    # LayerNorm at 16384); an odd row count keeps the general kernel where the layout has two row slots a workgroup
    assert lay(LB, 5120, BF) == (320, 2) and lay(RB, 5120, BF) == (320, 2)
    assert lay(LB, 7168, BF) == (448, 2) and lay(RB, 7168, BF, F32) == (448, 2)
    assert lay(LB, 14336, BF) == (896, 2) and lay(RB, 14336, BF) == (1024, 2)
    p = cabi.plan(LB, 16383, 5120, BF, BF)  # (one row slot a workgroup: any row count)
    assert (p["lanes_per_row"], p["packs_per_lane"], p["block_threads"]) == (320, 2, 320)
    p = cabi.plan(RB, 16383, 8192, BF, BF)
    assert (p["lanes_per_row"], p["packs_per_lane"], p["block_threads"]) == (512, 2, 512)
    p = cabi.plan(RB, 16383, 2048, BF, BF)  # two row slots and an odd row count: the general kernel
    assert (p["lanes_per_row"], p["packs_per_lane"], p["block_threads"]) == (128, 2, 512)
    p = cabi.plan(RB, 16384, 4096, BF, BF)
    assert (p["block_threads"], p["grid_blocks"], p["partial_rows"]) == (512, 256, 256)
    assert lay(LB, 3072, BF) == (256, 2) and lay(RB, 2560, BF) == (256, 2)  # which keeps its lanes below
    assert lay(LF, 3072, BF, F32) == (256, 2)                  # fp32 weights below 512 lanes
    assert lay(LF, 5120, BF, F32) == (320, 2) and lay(LF, 6144, BF, F32) == (256, 3)
    assert lay(cabi.OP_SOFTMAX_BWD, 5120, BF) == (512, 2)
    # 16-bit norm rows beyond 8192 elements: 512 lanes, not 1024
    assert lay(LF, 10240, BF) == (512, 3) and lay(LB, 10240, BF) == (512, 3)
    assert lay(RF, 12288, BF) == (512, 3) and lay(RB, 12288, BF) == (512, 3)
    assert lay(LF, 16384, BF) == (512, 4) and lay(LB, 16384, BF) == (1024, 2)
    assert lay(LB, 16384, cabi.F16, F32) == (1024, 2) and lay(LB, 12288, BF) == (512, 3)
    assert lay(RF, 16384, BF) == (512, 4) and lay(RB, 16384, BF) == (1024, 2)
    assert lay(LF, 32768, BF) == (1024, 4)
    # ragged 16-bit norm rows just above a power of two: three packs on half the lanes, except
    # in the LayerNorm backward (its three-pack kernels are over the registers of two workgroups)
    assert lay(LF, 4097, BF) == (256, 3) and lay(LB, 4097, BF) == (512, 2)
    assert lay(RB, 4097, BF) == (256, 3) and lay(RB, 2049, BF) == (128, 3)
    assert lay(LB, 2049, BF) == (256, 2) and lay(LB, 1025, BF) == (128, 2)
    assert lay(LB, 8193, BF) == (1024, 2) and lay(RB, 8193, BF) == (512, 3)
    # fp32 rows
    assert lay(LF, 5120, F32) == (512, 3) and lay(LB, 5120, F32) == (512, 3)
    assert lay(LF, 10240, F32) == (512, 5) and lay(RF, 10240, F32) == (1024, 3)
    assert lay(LB, 10240, F32) == (1024, 3) and lay(LB, 16384, F32) == (1024, 4)
    # ragged 16-bit softmax rows (the aligned window adds up to 7 elements in front)
    assert lay(cabi.OP_SOFTMAX_FWD, 4097, cabi.F16) == (256, 3)
    assert lay(cabi.OP_SOFTMAX_BWD, 4097, cabi.F16) == (256, 3)
    assert lay(cabi.OP_SOFTMAX_FWD, 4097, F32) == (512, 4)
    # ragged 16-bit norm rows: three packs in the forward and the RMSNorm backward
    assert lay(LF, 4097, cabi.F16) == (256, 3) and lay(RF, 4097, BF) == (256, 3)
    assert lay(RB, 4097, cabi.F16) == (256, 3) and lay(LB, 4097, cabi.F16) == (512, 2)


def test_group_norm_rows_take_512_lanes_while_two_workgroups_fit(cabi):
    """GroupNorm rows that would spread over 1024 lanes take 512 lanes with 6..10 (forward) or 6..7
    (backward) packs each; beyond that 1024 lanes with exactly the packs the row has."""
    BF, F32 = cabi.BF16, cabi.F32
    def lay(bwd, C, dt):  # [64, C, 64, 64] in 32 groups
        p = cabi.group_norm_plan(bwd, 64, C, 4096, 32, dt)
        return (p["lanes_per_row"], p["packs_per_lane"]) if p["resident"] else None
    assert lay(0, 160, BF) == (512, 5) and lay(1, 160, BF) == (512, 5)
    assert lay(0, 192, BF) == (512, 6) and lay(1, 192, BF) == (512, 6)
    assert lay(0, 224, BF) == (512, 7) and lay(1, 224, BF) == (512, 7)
    assert lay(0, 256, BF) == (512, 8) and lay(1, 256, BF) == (1024, 4)
    assert lay(0, 320, BF) == (512, 10) and lay(1, 320, F32) is None
    # (16-bit rows of exactly 512 x 10 packs in whole-wavefront channels: the exact kernels)
    assert lay(1, 320, BF) == (512, 10) and lay(1, 320, cabi.F16) == (512, 10)
    assert lay(0, 352, BF) == (1024, 6) and lay(1, 352, BF) == (1024, 6)
    assert lay(0, 96, F32) == (512, 6) and lay(1, 96, F32) == (512, 6)
    assert lay(0, 160, F32) == (512, 10) and lay(1, 128, F32) == (1024, 4)
    assert lay(0, 352, F32) == (1024, 11) and lay(0, 384, F32) is None and lay(1, 160, F32) is None


def test_forward_grid_grows_with_the_row_count(cabi):
    """The norm forward keeps a workgroup to about 2 (RMSNorm) / 4 (LayerNorm) row blocks, twice
    that with fp32 weights beside 16-bit rows, once the rows outgrow four resident grids; LayerNorm
    with fp32 weights beside 16-bit rows takes a grid of two or three resident workgroups a compute
    unit while that means at most 32 row blocks a workgroup."""
    BF, F32 = cabi.BF16, cabi.F32
    grid = lambda op, M, N, wd=BF: cabi.plan(op, M, N, BF, wd)["grid_blocks"]
    assert grid(cabi.OP_RMS_NORM_FWD, 16384, 2048) == 8192       # 256 CUs x 32: the floor
    assert grid(cabi.OP_LAYER_NORM_FWD, 16384, 2048) == 8192
    assert grid(cabi.OP_RMS_NORM_FWD, 16384, 6144, F32) == 768     # fp32 weights: three resident workgroups
    assert grid(cabi.OP_LAYER_NORM_FWD, 16384, 8192) == 512        # LayerNorm on 512 lanes: two
    assert grid(cabi.OP_RMS_NORM_FWD, 16384, 8192) == 8192
    assert grid(cabi.OP_LAYER_NORM_FWD, 16384, 8192, F32) == 512   # 256 CUs x two 512-thread workgroups
    assert grid(cabi.OP_LAYER_NORM_FWD, 16384, 6144, F32) == 768   # x three 256-thread workgroups
    assert grid(cabi.OP_LAYER_NORM_FWD, 300, 6144, F32) == 300     # never more workgroups than row blocks
    assert grid(cabi.OP_LAYER_NORM_FWD, 24576, 6144, F32) == 768   # 32 row blocks a workgroup: the last
    assert grid(cabi.OP_LAYER_NORM_FWD, 24577, 6144, F32) == 4096
    assert grid(cabi.OP_RMS_NORM_FWD, 65536, 6144) == 32768
    assert grid(cabi.OP_LAYER_NORM_FWD, 65536, 6144) == 16384
    assert grid(cabi.OP_LAYER_NORM_FWD, 65536, 6144, F32) == 8192
    # the exact layouts of 4096 / 5120 keep one resident grid up to 128 row blocks a workgroup
    assert grid(cabi.OP_LAYER_NORM_FWD, 300, 4096, F32) == 150
    assert grid(cabi.OP_RMS_NORM_FWD, 131072, 4096) == 512
    assert grid(cabi.OP_RMS_NORM_FWD, 262144, 4096) == 131072
    assert grid(cabi.OP_LAYER_NORM_FWD, 65536, 5120) == 768
    assert grid(cabi.OP_RMS_NORM_FWD, 262144, 2048) == 65536     # two rows a workgroup iteration
    assert grid(cabi.OP_RMS_NORM_BWD, 262144, 4096) == 256       # backward: one partial row each
    assert grid(cabi.OP_RMS_NORM_BWD, 262144, 6144) == 256
    assert grid(cabi.OP_RMS_NORM_BWD, 262144, 4096, F32) == 256
    assert cabi.plan(cabi.OP_RMS_NORM_BWD, 262144, 4096, F32, F32)["grid_blocks"] == 512


def test_forced_variants(cabi):
    cabi.set_override(cabi.OP_SOFTMAX_FWD, -1)
    assert cabi.plan(cabi.OP_SOFTMAX_FWD, 64, 2048, cabi.BF16, cabi.BF16)["resident"] == 0
    cabi.set_override(cabi.OP_SOFTMAX_FWD, 64, 1)  # 64 lanes x 1 pack cannot hold 2048 bf16
    with pytest.raises(RuntimeError, match="forced variant"):
        cabi.plan(cabi.OP_SOFTMAX_FWD, 64, 2048, cabi.BF16, cabi.BF16)
    cabi.clear_overrides()
    assert cabi.plan(cabi.OP_SOFTMAX_FWD, 64, 2048, cabi.BF16, cabi.BF16)["resident"] == 1


def test_strided_softmax_validation_and_plans(cabi):
    L = cabi.lib()
    one, null = ctypes.c_void_p(256), None
    f = L.mi355x_softmax_strided_fwd
    b = L.mi355x_softmax_strided_bwd
    assert f(one, one, 2, 3, 4, cabi.BF16, cabi.F32, 0, null) == -1       # only f16 -> f32
    assert f(one, one, 2, -1, 4, 0, 0, 0, null) == -2
    assert f(one, one, 2, 3, (1 << 30) + 1, 0, 0, 0, null) == -2
    assert f(one, one, 2, 3, 4, 0, 0, 3, null) == -2                       # unknown mode
    assert b(one, one, one, 2, 3, 4, 0, 0, cabi.SAFE_SOFTMAX, null) == -2  # no safe backward
    assert f(null, null, 2, 3, 4, 0, 0, 0, null) == -3
    assert b(one, null, one, 2, 3, 4, 0, 0, 0, null) == -3
    for dims in ((0, 3, 4), (2, 0, 4), (2, 3, 0)):
        assert f(null, null, *dims, 0, 0, 0, null) == 0
        assert b(null, null, null, *dims, 0, 0, 0, null) == 0
    for dt, E in ((cabi.F32, 4), (cabi.BF16, 8)):
        for outer in (1, 7, 4096):
            for D in (1, 2, 5, 32, 100, 256, 257, 2048, 100000):
                for inner in (2, 3, 8, 9, 100, 512, 513, 65536):
                    for bwd in (0, 1):
                        p = cabi.strided_plan(bwd, outer, D, inner, dt)
                        TX, TY, V = p["lanes_per_row"], p["rows_per_block"], p["packs_per_lane"]
                        assert 1 <= TX <= 64 and TX & (TX - 1) == 0 and TY & (TY - 1) == 0
                        assert TX * TY <= p["block_threads"] == 256
                        packs = -(-inner // E)
                        assert TX <= max(1, 1 << (packs - 1).bit_length())
                        tiles = outer * -(-packs // TX)
                        groups = 256 // (TX * TY)
                        assert 1 <= p["grid_blocks"] <= -(-tiles // groups)
                        if p["resident"]:
                            assert 1 <= V <= 8 and TY * V >= D > TY * (V - 1), "every row of D is held, none to spare"
                            if TX * TY > 64:  # more than a wavefront only when rows would get too short
                                assert TX <= 8
                        else:
                            assert D > 8 * 256 // min(4, 1 << (packs - 1).bit_length())
    # D = 256 fits the registers once the lanes along inner shrink to 8
    p = cabi.strided_plan(0, 4, 256, 4096, cabi.BF16)
    assert p["resident"] == 1 and p["lanes_per_row"] == 8 and p["packs_per_lane"] == 8
    # forced layouts that cannot hold D are refused
    cabi.set_override(cabi.OP_SOFTMAX_STRIDED_FWD, 64, 1)
    with pytest.raises(RuntimeError, match="forced variant"):
        cabi.strided_plan(0, 4, 5, 4096, cabi.BF16)
    cabi.set_override(cabi.OP_SOFTMAX_STRIDED_FWD, -1)
    assert cabi.strided_plan(0, 4, 5, 4096, cabi.BF16)["resident"] == 0
    cabi.clear_overrides()


def test_group_norm_validation_and_plans(cabi):
    L = cabi.lib()
    one, null = ctypes.c_void_p(256), None
    f = lambda N, C, HxW, G, xd=0, wd=0, x=one: L.mi355x_group_norm_fwd(x, null, null, one, null, null, N, C, HxW,
                                                                        G, 1e-5, xd, wd, null)
    assert f(2, 6, 4, 3, xd=cabi.F32, wd=cabi.BF16) == -1        # weights narrower than the rows
    assert f(2, 6, 4, 4) == -2                                   # C not a multiple of groups
    assert f(2, 6, 4, 0) == -2 and f(-1, 6, 4, 3) == -2
    assert f(1 << 30, 8, 4, 4) == -2                             # N * groups beyond 2^31
    assert f(1, 4, 1 << 30, 2) == -2                             # a group row beyond 2^30 elements
    assert f(0, 6, 4, 3, x=null) == 0 and f(2, 6, 0, 3, x=null) == 0 and f(2, 0, 4, 3, x=null) == 0
    assert f(2, 6, 4, 3, x=null) == -3
    b = L.mi355x_group_norm_bwd
    assert b(one, one, one, one, null, one, one, one, null, 0, 2, 6, 4, 3, 0, 0, null) == -4   # no workspace
    assert b(one, one, null, one, null, one, null, null, null, 0, 2, 6, 4, 3, 0, 0, null) == -3  # no mean
    assert b(one, one, one, one, null, null, null, null, null, 0, 2, 6, 4, 3, 0, 0, null) == 0  # nothing asked
    assert L.mi355x_group_norm_bwd_workspace_bytes(2, 6, 4, 3, 0, 0, 1, 0) == 2 * 2 * 6 * 4
    assert L.mi355x_group_norm_bwd_workspace_bytes(2, 6, 4, 3, 0, 0, 0, 0) == 0
    # rows too long for the registers need the channel sums for dX alone
    assert L.mi355x_group_norm_bwd_workspace_bytes(1, 4, 1 << 20, 2, 0, 0, 0, 0) == 2 * 1 * 4 * 4
    assert b(one, one, one, one, null, one, null, null, null, 0, 1, 4, 1 << 20, 2, 0, 0, null) == -4
    for dt, E in ((cabi.F32, 4), (cabi.BF16, 8)):
        for (N, C, HxW, G) in ((2, 4, 1, 2), (256, 32, 16, 4), (4, 64, 1024, 32), (2, 320, 4096, 32),
                               (3, 6, 5, 3), (1, 4, 1 << 17, 2), (1, 8, 1 << 20, 2),
                               # 7x7 and 14x14 maps: rows of whole packs, channels not
                               (4, 64, 49, 8), (2, 1024, 196, 32), (2, 128, 49, 2), (2, 130, 49, 2), (1, 1040, 49, 2),
                               (3, 8, 9, 1), (2, 16, 6, 2)):
            for bwd in (0, 1):
                p = cabi.group_norm_plan(bwd, N, C, HxW, G, dt)
                Lrow = (C // G) * HxW
                # 1: every pack in one channel; 2: rows of whole packs whose packs may straddle
                # two channels (needs a pack per channel at least and at most 512 channels a
                # group); 0: the general kernels
                kind = 1 if HxW % E == 0 else (2 if Lrow % E == 0 and HxW >= E and C // G <= 512 else 0)
                assert p["uniform"] == kind, (N, C, HxW, G, dt, p)
                assert p["grid_blocks"] >= 1
                if p["resident"]:
                    assert p["lanes_per_row"] * p["packs_per_lane"] * E >= Lrow
                    assert p["grid_blocks"] == -(-(N * G) // p["rows_per_block"])
                else:
                    assert Lrow > 8192
    # the diffusion-UNet shape keeps its 40960-element rows in registers
    assert cabi.group_norm_plan(0, 2, 320, 4096, 32, cabi.BF16)["resident"] == 1
    assert cabi.group_norm_plan(1, 2, 320, 4096, 32, cabi.BF16)["resident"] == 1


def test_plan_queries_of_empty_and_extreme_shapes(cabi):
    """The plan and workspace queries take any shape the entry points accept, empty ones included
    (the entry points return before they plan an empty call, the queries do not): no division by a
    zero row or tile count, and a shape beyond the limits is an error code, not a crash."""
    ops = (cabi.OP_LAYER_NORM_FWD, cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_FWD, cabi.OP_RMS_NORM_BWD,
           cabi.OP_SOFTMAX_FWD, cabi.OP_SOFTMAX_BWD)
    L = cabi.lib()
    for op in ops:
        for M, N in ((0, 0), (0, 4096), (0, 4194304), (5, 0), (0, 1), (1, 4194304), (3, 2 ** 30)):
            for dt in (cabi.F32, cabi.BF16):
                p = cabi.plan(op, M, N, dt, dt)
                assert p["grid_blocks"] >= 0 and p["block_threads"] > 0, (op, M, N, p)
        p = cabi.Plan()
        assert L.mi355x_rownorm_plan(op, 1, 2 ** 30 + 1, cabi.F32, cabi.F32, p) < 0
        assert L.mi355x_rownorm_plan(op, -1, 8, cabi.F32, cabi.F32, p) < 0
    for M, N in ((0, 0), (0, 4194304), (7, 0)):
        assert L.mi355x_layer_norm_bwd_workspace_bytes(M, N, cabi.BF16, cabi.BF16, 1, 1) == 0
        assert L.mi355x_rms_norm_bwd_workspace_bytes(M, N, cabi.BF16, cabi.BF16, 1) == 0
    for backward in (0, 1):
        for outer, D, inner in ((0, 8, 8), (4, 0, 8), (4, 8, 0), (0, 0, 0), (1, 8192, 8192)):
            p = cabi.strided_plan(backward, outer, D, inner, cabi.BF16)
            assert p["grid_blocks"] >= 0, (outer, D, inner, p)
        for N_, C, HxW in ((0, 32, 16), (4, 32, 0), (4, 0, 16)):
            p = cabi.group_norm_plan(backward, N_, C, HxW, 32 if C else 1, cabi.BF16)
            assert p["grid_blocks"] >= 0, (N_, C, HxW, p)
