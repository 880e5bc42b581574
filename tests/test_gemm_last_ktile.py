"""The slot schedule of a GEMM tile's last k-tile (the results leave under its MFMAs), replayed on the host:
every fragment is read before the MFMA that takes it and before the barrier that turns the operand buffers into
staging blocks, every accumulator block is complete before it is staged, every staged row is read back after its
last staging unit and stored after its read-back, and no slot of the read-back ring is overwritten while it
still holds a vector that has not been stored."""
import pytest

from lego_amd.kernels import gemm

# TM, TN, NPH, WN, block, MFMAs per slot of every tile built: 32x32x16 (and 32x32x64 for 8-bit) blocks one per slot,
# 16x16x32 blocks two per slot
SHAPES = [(4, 4, 4, 128, 32, 1), (2, 2, 4, 64, 32, 1), (2, 4, 4, 128, 32, 1), (4, 4, 2, 128, 32, 1), (2, 2, 2, 64, 32, 1),
          (4, 2, 4, 64, 32, 1), (8, 8, 2, 128, 16, 2), (4, 8, 2, 128, 16, 2), (4, 4, 2, 64, 16, 2)]


@pytest.mark.parametrize("TM,TN,NPH,WN,block,mps", SHAPES)
def test_last_ktile_schedule_is_a_valid_order(TM, TN, NPH, WN, block, mps):
    slots, tail = gemm.last_ktile_schedule(TM, TN, NPH, WN, block, mps)
    assert len(slots) == TM * TN * NPH // mps
    rows_per_it = block * WN // 512                          # read-backs per block row
    units_per_block = block * block // 256
    have = {(0, f) for f in range(TM + TN)}                  # fragments of k-step 0 arrive with the tile
    done = {}                                                # block -> k-steps summed
    events = []
    final_slot = {}
    barrier_at = None
    for g, slot in enumerate(slots):
        for ks, f in slot["loads"]:
            assert barrier_at is None, "a fragment read after the operand buffers were handed over"
            assert 0 < ks < NPH and 0 <= f < TM + TN and (ks, f) not in have
            have.add((ks, f))
        assert len(slot["mfmas"]) == mps
        for i, j, ks in slot["mfmas"]:
            assert (ks, i) in have and (ks, TM + j) in have, f"slot {g}: fragment not read yet"
            assert done.get((i, j), 0) == ks                 # k-steps of a block in order
            done[(i, j)] = ks + 1
            final_slot[(i, j)] = g
        for i2, j2, q in slot["stage"]:
            assert barrier_at is not None and done.get((i2, j2), 0) == NPH, f"slot {g}: block ({i2}, {j2}) staged early"
            # (a whole slot of MFMAs lies between an inline-assembly MFMA and the read of its result)
            assert mps == 1 or g - final_slot[(i2, j2)] >= 2
            events.append(("stage", (i2, j2, q)))
        events += [("rb", it) for it in slot["rb"]] + [("st", it) for it in slot["st"]]
        if slot["barrier"]:
            assert barrier_at is None
            barrier_at = g
    assert len(have) == NPH * (TM + TN) and all(v == NPH for v in done.values()) and len(done) == TM * TN
    # MFMAs as inline assembly (more than one per slot): a fence (with the wait states of an MFMA) stands between
    # the last slot and the first read of one of its results
    last_slot_blocks = {(i, j) for i, j, ks in slots[-1]["mfmas"] if ks == NPH - 1}
    staged_in_tail = [u[:2] for kind, u in tail if kind == "stage"]
    if mps > 1:
        at = [kind for kind, u in tail].index("fence")
        before = [u[:2] for kind, u in tail[:at] if kind == "stage"]
        assert not last_slot_blocks & set(before)
        assert last_slot_blocks <= set(staged_in_tail)
    else:
        assert all(kind != "fence" for kind, u in tail)
    tail = [(kind, u) for kind, u in tail if kind != "fence"]
    events += [(kind, tuple(u) if kind == "stage" else u) for kind, u in tail]
    units = [u for kind, u in events if kind == "stage"]
    assert sorted(units) == sorted((i, j, q) for i in range(TM) for j in range(TN) for q in range(units_per_block))
    for kind in ("rb", "st"):
        assert sorted(u for k, u in events if k == kind) == list(range(TM * rows_per_it))
    in_flight = {}
    for n, (kind, u) in enumerate(events):
        if kind == "rb":
            row = u // rows_per_it
            last_unit = max(m for m, (k, v) in enumerate(events) if k == "stage" and v[0] == row)
            assert last_unit < n, f"row {row} read back before it is staged"
            ring = u % gemm.LAST_KTILE_RING
            assert ring not in in_flight, f"ring slot {ring} overwritten while vector {in_flight.get(ring)} waits"
            in_flight[ring] = u
        elif kind == "st":
            assert in_flight.pop(u % gemm.LAST_KTILE_RING, None) == u, f"vector {u} stored before it is read back"
    assert not in_flight


def test_staging_offsets_split_into_lane_and_unit_constants():
    """The cheap addressing of the staging block (one XOR with a literal and an immediate per access) is the
    layout's own offset: spot-check the constants the generator derived against the printed expressions."""
    p = gemm._tile_params(256, 256, 64, (2, 2), 8, False, False, True, "f16")

    def cexpr(text, **env):
        import re
        return eval(re.sub(r"\(\((\w+)\)/\((\d+)\)\)", r"(\1//\2)", text), {"__builtins__": {}}, env)
    seen = 0
    for slot in p["last_slots"]:
        for i, j, q, add, xor in slot["stage"]:
            for l32 in (0, 5, 31):
                for lhi in (0, 1):
                    want = cexpr(p["c_stage_store"], i=i, j=j, q=q, l32=l32, lhi=lhi)
                    assert want == add + (cexpr(p["c_stage_lane"], l32=l32, lhi=lhi) ^ xor)
                    seen += 1
        for it, add, xor in slot["rb"]:
            for lane in (0, 17, 63):
                cr, cp = cexpr(p["c_out_row"], it=it, lane=lane), cexpr(p["c_out_pair"], it=it, lane=lane)
                assert cexpr(p["c_stage_load"], cr=cr, cp=cp) == add + (cexpr(p["c_back_lane"], lane=lane) ^ xor)
                seen += 1
    assert seen > 300


def test_build_check_finds_an_accumulator_read_close_behind_an_inline_assembly_mfma():
    """The build reads the device assembly of every unit whose MFMAs are inline assembly: the checker behind it, on
    two listings -- a result read three instructions after its MFMA, and one read after twenty."""
    from lego_amd import build
    mfma = "\tv_mfma_f32_16x16x32_f16 a[4:7], v[2:5], v[6:9], a[4:7]\n"
    other = "\tv_add_u32_e32 v1, v2, v3\n"
    head = "\t.text\nkernel_a:\n; %bb.0:\n"
    close = head + mfma + other * 2 + "\tv_accvgpr_read_b32 v10, a5\n\ts_endpgm\n"
    far = head + mfma + "\tv_mfma_f32_16x16x32_f16 a[0:3], v[2:5], v[6:9], a[0:3]\n" + other * 19 + \
        "\tv_accvgpr_read_b32 v10, a[4:5]\n\ts_endpgm\nkernel_b:\n" + mfma + "\ts_endpgm\n"
    assert build.asm_mfma_read_distance(close) == {"kernel_a": (3, 5, "v_accvgpr_read_b32")}
    found = build.asm_mfma_read_distance(far)
    assert found == {"kernel_a": (24, 4, "v_accvgpr_read_b32")}      # an MFMA between counts four; kernel_b reads nothing back
    assert found["kernel_a"][0] >= build.ASM_MFMA_MIN_DISTANCE > 3

