"""The slot schedule of a GEMM tile's last k-tile (the results leave under its MFMAs), replayed on the host:
every fragment is read before the MFMA that takes it and before the barrier that turns the operand buffers into
staging blocks, every accumulator block is complete before it is staged, every staged row is read back after its
last staging unit and stored after its read-back, and no slot of the read-back ring is overwritten while it
still holds a vector that has not been stored."""
import pytest

from lego_amd.kernels import gemm

SHAPES = [(4, 4, 4, 128), (2, 2, 4, 64), (2, 4, 4, 128), (4, 4, 2, 128), (2, 2, 2, 64)]      # TM, TN, NPH, WN of every tile built


@pytest.mark.parametrize("TM,TN,NPH,WN", SHAPES)
def test_last_ktile_schedule_is_a_valid_order(TM, TN, NPH, WN):
    slots, tail = gemm.last_ktile_schedule(TM, TN, NPH, WN)
    assert len(slots) == TM * TN * NPH
    rows_per_it = WN // 16                                   # read-backs per block row of 32 rows
    have = {(0, f) for f in range(TM + TN)}                  # fragments of k-step 0 arrive with the tile
    done = {}                                                # block -> k-steps summed
    events = []
    barrier_at = None
    for g, slot in enumerate(slots):
        for ks, f in slot["loads"]:
            assert barrier_at is None, "a fragment read after the operand buffers were handed over"
            assert 0 < ks < NPH and 0 <= f < TM + TN and (ks, f) not in have
            have.add((ks, f))
        i, j, ks = slot["mfma"]
        assert (ks, i) in have and (ks, TM + j) in have, f"slot {g}: fragment not read yet"
        assert done.get((i, j), 0) == ks                     # k-steps of a block in order
        done[(i, j)] = ks + 1
        for i2, j2, q in slot["stage"]:
            assert barrier_at is not None and done.get((i2, j2), 0) == NPH, f"slot {g}: block ({i2}, {j2}) staged early"
            events.append(("stage", (i2, j2, q)))
        events += [("rb", it) for it in slot["rb"]] + [("st", it) for it in slot["st"]]
        if slot["barrier"]:
            assert barrier_at is None
            barrier_at = g
    assert len(have) == NPH * (TM + TN) and all(v == NPH for v in done.values()) and len(done) == TM * TN
    events += [(kind, tuple(u) if kind == "stage" else u) for kind, u in tail]
    units = [u for kind, u in events if kind == "stage"]
    assert sorted(units) == sorted((i, j, q) for i in range(TM) for j in range(TN) for q in range(4))
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
