"""Which kernel each benchmark shape is dispatched to (kvmix_quantized_gemv_plan: no launch, no GPU).

A change of the dispatch rules that moves one of the measured shapes onto another kernel (the
generic fallback above all) has to show up here, not only as a slower bench line.
"""
import ctypes

import pytest

from kvmix_amd import _lib

REF, DENSE3 = _lib.FMT_REF, _lib.FMT_DENSE3


def plan(bits, fmt, batch, kv_heads, rep, tokens, head_dim, side, group=32):
    """side 'qk': x is the query (K = head_dim rows, N = tokens); 'pv': x is a row of probabilities."""
    samples = batch * kv_heads * rep
    if bits == 3 and fmt == REF:
        group = 11
    if side == "qk":
        return _lib.gemv_plan(group, bits, fmt, samples, rep, 1, head_dim, tokens)
    return _lib.gemv_plan(group, bits, fmt, samples, rep, 1, tokens, head_dim)


@pytest.mark.parametrize("bits", [2, 4])
def test_target_shape_b16_t8k(bits):
    # 2/4-bit Llama-2-7B KV at 8k context, batch 16 (8064 quantized tokens + the fp16 window)
    qk = plan(bits, REF, 16, 32, 1, 8064, 128, "qk")
    # the wide tiles (2048 codes per wave): four waves cover a row, 2048 waves in all = one round at two per SIMD
    assert qk["kernel"] == f"gemv_cols_mfma2<{bits},1,1>" and qk["launches"] == 1
    assert qk["grid"][:2] == (1, 512) and qk["block"] == (64, 4, 1)
    pv = plan(bits, REF, 16, 32, 1, 8064, 128, "pv")
    assert pv["kernel"] == f"gemv_rows_mfma<{bits},1,1>" and pv["launches"] == 1 and pv["splits"] == 1


def test_config0_single_layer_b1_t4096():
    qk = plan(4, REF, 1, 32, 1, 3968, 128, "qk")
    assert qk["kernel"].startswith("gemv_cols_mfma2<4,")
    pv = plan(4, REF, 1, 32, 1, 3968, 128, "pv")
    # 32 slices: one block of sixteen waves each, no second launch for a reduction
    assert pv["kernel"] == "gemv_rows_mfma<4,1,1>" and pv["block"] == (64, 16, 1) and pv["launches"] == 1


def test_config1_mixed_bits_b8_t8192():
    # one round of the plain tiles (1024 codes per wave) covers these launches
    assert plan(4, REF, 8, 32, 1, 8064, 128, "qk")["kernel"] == "gemv_cols_mfma2<4,1,0>"
    assert plan(2, REF, 8, 32, 1, 8064, 128, "qk")["kernel"] == "gemv_cols_mfma2<2,1,0>"
    # large batches: 2 bits stay on the matrix cores with the wide tiles, 4 bits go to the vector-ALU kernel
    assert plan(2, REF, 32, 32, 1, 8064, 128, "qk")["kernel"].startswith("gemv_cols_mfma2<2,") and \
        plan(2, REF, 32, 32, 1, 8064, 128, "qk")["kernel"].endswith(",1>")
    assert plan(4, REF, 32, 32, 1, 8064, 128, "qk")["kernel"].startswith("gemv_cols<4,")
    # the reference's 3-bit keys: 11 codes a word, 8063 = 733 * 11 tokens
    ref3 = plan(3, REF, 8, 32, 1, 8063, 128, "qk")
    # 256 rows of three 256-word tiles: a block per row, a wave per tile that walks all channel rows -- one block on
    # every CU
    assert ref3["kernel"] == "gemv_cols3<1,4,8,1>" and ref3["ksplit"] == 1 and ref3["grid"][:2] == (1, 256)
    assert ref3["block"] == (64, 3, 1)
    # one row more than there are CUs, or a longer row: 128-word tiles, four waves a tile, each with a quarter of
    # the channel rows
    ref3 = plan(3, REF, 9, 32, 1, 8063, 128, "qk")
    assert ref3["kernel"] == "gemv_cols3<2,4,8,1>" and ref3["ksplit"] == 4 and ref3["grid"][:2] == (6, 288)
    ref3 = plan(3, REF, 8, 32, 1, 1477 * 11, 128, "qk")
    assert ref3["kernel"] == "gemv_cols3<2,4,8,1>" and ref3["ksplit"] == 4
    # ... and again whole rows where they make three blocks of four waves per CU
    assert plan(3, REF, 8, 32, 1, 2967 * 11, 128, "qk")["kernel"] == "gemv_cols3<1,4,8,1>"
    assert plan(3, DENSE3, 8, 32, 1, 8064, 128, "qk")["kernel"].startswith("gemv_cols<30,")
    for bits, mode in ((4, 4), (2, 2)):
        assert plan(bits, REF, 8, 32, 1, 8064, 128, "pv")["kernel"] == f"gemv_rows_mfma<{mode},1,1>"
    assert plan(3, DENSE3, 8, 32, 1, 8064, 128, "pv")["kernel"] == "gemv_rows_mfma<30,1,1>"


def test_config2_gqa_b16_t32k():
    # four query heads share a key/value head: one block serves all four from one pass over the codes
    qk = plan(3, REF, 16, 8, 4, 32637, 128, "qk")
    assert qk["kernel"].startswith("gemv_cols3<") and qk["kernel"].endswith(",4>")
    assert qk["grid"][1] == 16 * 8
    pv = plan(2, REF, 16, 8, 4, 32640, 128, "pv")
    assert pv["kernel"] == "gemv_rows_mfma<2,4,1>" and pv["grid"][1] == 16 * 8


@pytest.mark.parametrize("batch", [1, 16, 64, 128])
@pytest.mark.parametrize("bits", [1, 2])
def test_config3_sweep_t4096_residual32(bits, batch):
    qk = plan(bits, REF, batch, 32, 1, 4064, 128, "qk")["kernel"]
    if bits == 1 and batch <= 16:
        assert qk == "gemv_cols_mfma<1,1>"   # several tiles per wave: ahead while one round of waves covers the launch
    else:
        # non-temporal code loads (second argument) for 2-bit launches of up to three resident rounds of waves
        assert qk.startswith(f"gemv_cols_mfma2<{bits},{int(bits == 2 and batch <= 64)},")
    assert plan(bits, REF, batch, 32, 1, 4064, 128, "pv")["kernel"] == f"gemv_rows_mfma<{bits},1,1>"


def test_only_odd_shapes_reach_the_generic_kernel():
    assert plan(4, REF, 2, 4, 1, 96, 128, "qk")["kernel"] == "gemv_generic<4>"   # three groups a row
    assert plan(4, REF, 2, 4, 1, 4, 128, "pv")["kernel"] == "gemv_generic<4>"    # four rows
    assert plan(4, REF, 2, 4, 1, 8064, 128, "qk", group=64)["kernel"] == "gemv_generic<4>"
    empty = plan(4, REF, 2, 4, 1, 0, 128, "pv")
    assert empty["launches"] <= 1


def test_batches_beyond_a_grid_dimension_go_out_in_parts():
    p = _lib.gemv_plan(32, 4, REF, 70000, 1, 1, 16, 64)
    assert p["launches"] == 2 and p["grid"][1] == 35000
    p = _lib.gemv_plan(32, 4, REF, 3 * 65536, 4, 1, 256, 128)        # whole kv heads (four query heads) per part
    assert p["launches"] == 4 and p["grid"][1] * 4 * 4 == 3 * 65536
    assert _lib.load().kvmix_gemv_workspace_bytes(70000, 1, 4096, 128) == 0


def test_plan_reports_the_call_s_own_errors():
    p = _lib.GemvPlan()
    L = _lib.load()
    assert L.kvmix_quantized_gemv_plan(32, 5, 0, 1, 1, 1, 128, 128, 16, 4, ctypes.byref(p)) == -1   # KVMIX_ERR_BITS
    assert L.kvmix_quantized_gemv_plan(32, 4, 0, 1, 1, 1, 128, 100, 16, 4, ctypes.byref(p)) == -3   # ..._STEPS_GROUP
    assert L.kvmix_quantized_gemv_plan(32, 4, 0, 1, 1, 1, 128, 128, 8, 4, ctypes.byref(p)) == -8    # ..._SHAPE
    assert L.kvmix_quantized_gemv_plan(32, 4, 0, 1, 1, 1, 128, 128, 16, 4, None) == -7              # ..._NULL


# tile widths (in group units along N) of the tiled q.K^T kernels, from their names: a tile must fit into the row
def _tile_units(kernel):
    import re

    m = re.match(r"gemv_cols3<(\d+),(\d+),", kernel)
    if m:
        return (64 // int(m.group(1))) * int(m.group(2))
    m = re.match(r"gemv_cols<(\d+),(\d+),(\d+)>", kernel)
    if m:
        return (64 // int(m.group(2))) * int(m.group(3))
    m = re.match(r"gemv_cols_mfma2<(\d+),(\d+),(\d+)>", kernel)
    if m:
        return 64 if int(m.group(3)) else 32   # (third argument: the wide tiles)
    if kernel.startswith("gemv_cols_mfma<"):
        return 16
    return 0


def test_no_shape_is_given_a_kernel_whose_tile_is_wider_than_the_row():
    """A sweep of q.K^T and p.V problems through the dispatch (no launch): every one is accepted -- a launcher
    that found its kernel's tile wider than the row, or its chunk longer than K, would make the query fail --
    and the kernel named covers the row with whole tiles that fit into it."""
    checked = 0
    for bits, fmt, group, unit in ((1, REF, 32, 32), (2, REF, 32, 32), (4, REF, 32, 32), (3, REF, 11, 11), (3, DENSE3, 32, 32)):
        for rep in (1, 4, 8):
            for batch in (1, 2, 8, 64, 700):
                samples = batch * 2 * rep
                for units in (1, 2, 7, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 209, 255, 256, 257, 511, 733, 1024, 2978, 9000):
                    tokens = units * unit
                    for head_dim in (16, 64, 128, 256):
                        p = _lib.gemv_plan(group, bits, fmt, samples, rep, 1, head_dim, tokens)      # q.K^T
                        tu = _tile_units(p["kernel"])
                        assert tu <= units, (p["kernel"], bits, fmt, samples, rep, head_dim, tokens)
                        if p["kernel"].startswith("gemv_cols_mfma"):
                            assert head_dim >= (16 if "mfma2" in p["kernel"] else 32)
                        if fmt == REF and bits == 3:
                            continue  # (values are never in the reference's 3-bit key format here)
                        if head_dim % 32 == 0 and tokens % 8 == 0:
                            q = _lib.gemv_plan(32, bits, fmt, samples, rep, 1, tokens, head_dim)     # p.V
                            if q["kernel"].startswith("gemv_rows_mfma"):
                                assert tokens >= 128, (q["kernel"], tokens)
                        checked += 1
    assert checked > 5000


# ---- the single-pass attention step's plan (kvmix_decode_attention_fused_plan: no launch, no GPU) ----

def _step(batch, heads, kv_heads, k_bits, k_fmt, k_tokens, v_bits, v_fmt, v_tokens, width, **kw):
    k_group = 11 if (k_bits == 3 and k_fmt == REF) else 32
    return _lib.attn_step_descriptor(batch, heads, kv_heads, 128, k_bits, k_fmt, k_group, k_tokens, v_bits, v_fmt, 32,
                                     v_tokens, width - k_tokens, width - v_tokens, **kw)


def test_attention_step_plans_of_the_measured_shapes():
    # B = 16, T = 8192, 4-bit keys and values: matrix cores over [0, 8064) (two blocks of four tiles per query head),
    # the two 128-token fp16 tails as one slab of 256 positions in a trailing block of the same launch, and the merge
    p = _lib.attn_plan(_step(16, 32, 32, 4, REF, 8064, 4, REF, 8064, 8192))
    assert p["matrix"] and p["matrix_tiles"] == 8 and p["slab_begin"] == 8064 and p["launches"] == 2
    assert (p["slabs"], p["slab_positions"], p["slab_blocks"]) == (1, 256, 512)
    assert p["matrix_grid"] == (2 * 512 + 512, 1, 1) and p["matrix_block"] == (64, 4, 1)
    # keys and values quantized to different lengths: tiles over what both have, slabs over the rest
    p = _lib.attn_plan(_step(16, 32, 32, 2, REF, 8064, 4, REF, 7968, 8192))
    assert p["matrix"] and p["slab_begin"] == 7968 and p["slabs"] == 1 and p["launches"] == 2
    # the reference's 3-bit keys (733 words = 8063 tokens) with 2-bit values (8064): tiles of 1408 positions over
    # [0, 7744) = 22 * 352, two slabs of 352 over the remaining quantized positions and the tails
    p = _lib.attn_plan(_step(8, 32, 32, 3, REF, 8063, 2, REF, 8064, 8192))
    assert p["matrix"] and (p["matrix_tiles"], p["slab_begin"], p["slab_positions"], p["slabs"]) == (6, 7744, 352, 2)
    assert p["matrix_grid"][0] == 2 * 256 + 2 * 256 and p["launches"] == 2
    assert p["matrix_tile_waves"] == 1
    # configs[4]'s size: few (query head, tile) pairs, so the four waves of a block share a tile (a block per tile)
    p = _lib.attn_plan(_step(4, 32, 32, 4, REF, 2176, 4, REF, 2176, 2304))
    assert p["matrix"] and p["matrix_tile_waves"] == 4 and p["matrix_tiles"] == 3 and p["slab_begin"] == 2176
    assert p["matrix_grid"][0] == 3 * 128 + 128 and p["slabs"] == 1 and p["launches"] == 2 and p["recommended"]
    # ... also with the reference's 3-bit keys from 128 pairs on (2167 -> 2112 = 6 * 352 positions, two tiles of 1408)
    p = _lib.attn_plan(_step(4, 32, 32, 3, REF, 2167, 2, REF, 2176, 2304))
    assert p["matrix"] and p["matrix_tile_waves"] == 4 and p["matrix_tiles"] == 2 and p["slab_begin"] == 2112
    p = _lib.attn_plan(_step(1, 32, 32, 3, REF, 2167, 2, REF, 2176, 2304))
    assert not p["matrix"] and p["slab_begin"] == 0 and p["slabs"] == 4 and p["launches"] == 2
    # under one tile of quantized positions: the vector-ALU slab kernel from position 0
    p = _lib.attn_plan(_step(4, 32, 32, 4, REF, 896, 4, REF, 896, 1024))
    assert not p["matrix"] and p["matrix_tile_waves"] == 0 and p["slab_begin"] == 0 and p["slabs"] == 2 and p["launches"] == 2
    # one slab: the slab kernel stores the result itself
    p = _lib.attn_plan(_step(8, 32, 32, 2, REF, 384, 2, REF, 384, 512))
    assert not p["matrix"] and p["slabs"] == 1 and p["launches"] == 1


def test_no_attention_step_is_given_a_tile_longer_than_its_quantized_part():
    """A sweep of step sizes through the plan query: wherever the matrix-core kernel is chosen, its 1024-position
    tiles fit into the quantized part, that part is whole groups, the grid covers every tile with no more than
    65535 rows, and the vector-ALU slabs cover every position from where the tiles end."""
    checked = 0
    for k_bits, k_fmt in ((1, REF), (2, REF), (4, REF), (3, REF), (3, DENSE3)):
        unit = 11 if (k_bits == 3 and k_fmt == REF) else 32
        for v_bits, v_fmt in ((1, REF), (2, REF), (4, REF), (3, DENSE3)):
            for batch, heads, kv_heads in ((1, 32, 32), (4, 32, 8), (16, 32, 32), (64, 32, 32), (2100, 32, 32)):
                for units in (0, 1, 3, 31, 32, 33, 63, 64, 93, 252, 1000):
                    for tail in (0, 1, 32, 128):
                        for dv in (0, 32, -32):
                            k_tokens = units * unit
                            v_tokens = max(k_tokens // 32 * 32 + dv, 0) if unit == 32 else max((k_tokens + tail) // 32 * 32 + dv, 0)
                            width = max(k_tokens, v_tokens) + tail
                            if width == 0:
                                continue
                            st = _step(batch, heads, kv_heads, k_bits, k_fmt, k_tokens, v_bits, v_fmt, v_tokens, width)
                            plan = _lib.AttnPlan()
                            rc = _lib.load().kvmix_decode_attention_fused_plan(ctypes.byref(st), ctypes.byref(plan))
                            if batch * heads * ((width + 511) // 512) > 0x7fffffff:
                                assert rc == -8
                                continue
                            assert rc == 0, (rc, k_bits, k_fmt, v_bits, batch, k_tokens, v_tokens, width)
                            if plan.matrix:
                                # tiles of 1024 positions over what both sides have quantized; with the reference's
                                # 3-bit keys tiles of 1408 over whole multiples of lcm(11, 32) = 352
                                step, tile = (352, 1408) if unit == 11 else (32, 1024)
                                both = min(k_tokens, v_tokens) // step * step
                                assert both >= tile and (k_fmt, k_bits) != (DENSE3, 3)
                                assert plan.slab_begin == both and plan.matrix_tiles == (both + tile - 1) // tile
                                assert plan.slab_positions == (352 if unit == 11 else 256)
                                blocks_per_head = (plan.matrix_grid[0] - plan.slab_blocks) // (batch * heads)
                                assert plan.matrix_tile_waves in (1, 4) and plan.matrix_block[1] == 4
                                # a wave per tile (blocks of four tiles) or a block per tile
                                assert blocks_per_head * (4 // plan.matrix_tile_waves) >= plan.matrix_tiles
                                assert (blocks_per_head - 1) * (4 // plan.matrix_tile_waves) < plan.matrix_tiles
                                assert plan.matrix_grid[0] == blocks_per_head * batch * heads + plan.slabs * batch * heads
                            else:
                                assert plan.slab_begin == 0 and plan.matrix_tiles == 0 and plan.matrix_tile_waves == 0
                            assert plan.slab_begin + plan.slabs * plan.slab_positions >= width
                            checked += 1
    assert checked > 5000


def test_committed_traffic_figures_belong_to_the_kernels_the_step_runs():
    """profiles/hbm_traffic.json carries, beside every HBM-traffic figure bench.py quotes as roofline.traffic, the
    device kernel it was measured on; the bench drops a figure whose kernel the dispatch no longer picks.  Here:
    the committed file is current -- every GEMV of the bench step (B = 8, T = 8192, R = 128) still gets that kernel."""
    import json
    import os
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.path.insert(0, root)
    import bench

    tj = json.load(open(os.path.join(root, "profiles", "hbm_traffic.json")))
    names = tj["_kernels"]
    gemvs = [t for t in names if t.startswith("gemv")]
    assert sorted(gemvs) == sorted(t for t in tj if t.startswith("gemv"))
    for tag in gemvs:
        assert bench.device_kernel(_lib, tag, 8, 32, 128, 8192 - 128) == names[tag], tag
