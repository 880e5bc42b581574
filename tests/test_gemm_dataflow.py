"""CPU simulation of the GEMM kernels' data movement, from the generated text itself.

The address expressions are taken out of the emitted HIP source and evaluated for every lane:
where each memory->LDS instruction puts which bytes of the operand tile, and which bytes the
fragment reads hand to each lane -- including the transposing LDS reads, simulated with the
lane/element rule measured on gfx950:

* ``ds_read_b64_tr_b16``: within a group of 16 lanes, lane ``i`` receives element ``i % 4`` of
  source lanes ``i//4 + 4*j``, ``j = 0..3``;
* ``ds_read_b64_tr_b8``: lane ``i`` receives byte ``i % 8`` of source lanes ``i//8 + 2*j``,
  ``j = 0..7``.

Expected: lane ``l`` of an MFMA operand holds row/column ``l % block`` and the ``k``-values
``(l // block) * kk .. + kk - 1`` of the k-step, ``kk`` = 8 (16-bit) or 32 (8-bit), in order; ``block`` = 32 for
the 32x32 MFMAs (a k-step of 2 kk), 16 for v_mfma_f32_16x16x32 (a k-step of 4 kk).
"""
import re

import numpy as np
import pytest

from lego_amd.kernels import gemm


def _c_eval(expr, env):
    """Evaluate a printed C index expression (non-negative integers: ``/`` is floor division)."""
    return eval(expr.replace("/", "//"), {"__builtins__": {}}, env)


def _grab(text, pattern):
    m = re.search(pattern, text)
    assert m, pattern
    return m.group(1)


def _args(call):
    """Top-level comma-separated arguments of ``name(arg, arg, ...)``."""
    inner = call[call.index("(") + 1:call.rindex(")")]
    out, depth, cur = [], 0, ""
    for ch in inner:
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
            continue
        depth += ch == "("
        depth -= ch == ")"
        cur += ch
    return out + [cur]


@pytest.mark.parametrize("dtype,bk,tile,block", [("f16", 64, 256, 32), ("f16", 64, 256, 16), ("e5m2", 128, 256, 32),
                                                 ("f16", 64, 128, 32)])
@pytest.mark.parametrize("variant", ["nn", "tt"])
def test_fragments_receive_the_right_elements(dtype, bk, tile, block, variant):
    ta, tb = variant[0] == "t", variant[1] == "t"
    unit, _ = gemm.emit(bm=tile, bn=tile, bk=bk, trans_a=ta, trans_b=tb, with_grouped=False, dtype=dtype, block=block)
    text = unit.text
    esize = 2 if dtype == "f16" else 1
    epc = 16 // esize                       # elements per 16-byte chunk
    kk = 8 if esize == 2 else 32            # k-values a lane holds per MFMA
    M = N = 512
    K = 2 * bk
    sizes = dict(M=M, N=N, K=K)
    for role, rows_total, kmajor in (("a", M, not ta), ("b", N, tb)):
        src0 = _grab(text, r"const unsigned %s_src0 = \d \* \((.*)\);" % role)
        step = _grab(text, r"%s_src_step = \d \* \((.*?)\)[,;]" % role)
        # (the lane's offset for odd instructions, where the LDS layout's key changes with the instruction's parity)
        odd = re.search(r"const unsigned %s_src0_odd = \d \* \((.*)\);" % role, text)
        src0_odd = odd.group(1) if odd else src0
        iters = tile * bk // epc // 256
        # --- what the memory->LDS instructions leave in the LDS buffer: element ids of tile (0, 0)
        lds = np.full(tile * bk, -1, dtype=np.int64)
        for wave in range(4):
            for lane in range(64):
                bases = [_c_eval(e, dict(sizes, wave=wave, lane=lane)) for e in (src0, src0_odd)]
                for it in range(iters):
                    off = bases[it % 2] + it * _c_eval(step, sizes)          # element offset inside the operand
                    slot = (it * 4 + wave) * 64 + lane
                    # element id = (row, k) of the tile: k-major storage has pitch K, the other pitch rows_total
                    for e in range(epc):
                        if kmajor:
                            r_, k_ = divmod(off + e, K)
                        else:
                            k_, r_ = divmod(off + e, rows_total)
                        assert 0 <= r_ < tile and 0 <= k_ < bk
                        assert lds[slot * epc + e] == -1
                        lds[slot * epc + e] = r_ * bk + k_
        assert (lds >= 0).all() and len(set(lds.tolist())) == tile * bk    # the whole tile, once
        # --- what the fragment reads hand to the lanes
        frag = _grab(text, r"f%s\[BUF\]\[%s\] = (.*?); \}" % (role, "i" if role == "a" else "j"))
        groups = 64 // block                        # lane groups of an operand, kk k-values each
        for ks in range(bk // (groups * kk)):
            for sub in range(tile // 2 // block):
                for w in range(2):
                    env0 = dict(ks=ks, i=sub, j=sub, wm=w, wn=w)
                    want_row0 = w * (tile // 2) + sub * block

                    def addr(expr, lane):
                        env = dict(env0, l32=lane % 32, lhi=lane // 32, l16=lane % 16, lgrp=lane // 16)
                        return _c_eval(expr, env)

                    got = np.zeros((64, kk), dtype=np.int64)
                    if kmajor:
                        ptrs = [frag[frag.index("+ (") + 2:frag.rindex(")")]] if esize == 2 else \
                            [a[a.index("+ (") + 2:] for a in _args(frag)]
                        for lane in range(64):
                            vals = []
                            for pexp in ptrs:
                                p0 = addr(pexp, lane)
                                assert p0 % epc == 0
                                vals += lds[p0:p0 + epc].tolist()
                            got[lane] = vals
                    else:
                        ptrs = [a[a.index("+ (") + 2:] for a in _args(frag)]
                        per = 8 // esize                         # elements per 8-byte read
                        for r, pexp in enumerate(ptrs):
                            for lane in range(64):
                                g, i_ = lane // 16, lane % 16
                                for jj in range(per):
                                    src = 16 * g + i_ // per + (16 // per) * jj
                                    p0 = addr(pexp, src)
                                    assert p0 % per == 0
                                    got[lane, r * per + jj] = lds[p0 + i_ % per]
                    for lane in range(64):
                        row = want_row0 + lane % block
                        k0 = ks * groups * kk + (lane // block) * kk
                        assert got[lane].tolist() == [row * bk + k0 + x for x in range(kk)], (role, ks, sub, w, lane)


@pytest.mark.parametrize("tile,block", [(256, 32), (256, 16), (128, 32)])
@pytest.mark.parametrize("variant", ["nn", "nt", "tn", "tt"])
def test_ragged_edges_skip_exactly_what_lies_outside(variant, tile, block):
    """The EDGE instantiation runs memory->LDS instruction ``x`` under the mask of the lanes with
    ``edge0 + x*step < rem``.  For a tile with ``rem`` valid rows (columns), replay the masks: every chunk that
    passes must lie inside the operand, and every chunk with data of a valid row (column) must pass."""
    ta, tb = variant[0] == "t", variant[1] == "t"
    bk = 64
    unit, _ = gemm.emit(bm=tile, bn=tile, bk=bk, trans_a=ta, trans_b=tb, with_grouped=False, block=block)
    text = unit.text
    K = 2 * bk
    edge_odds = re.search(r"const unsigned a_edge0_odd = (.*), b_edge0_odd = (.*);", text).groups()
    for role, kmajor in (("a", not ta), ("b", tb)):
        src0 = _grab(text, r"const unsigned %s_src0 = \d \* \((.*)\);" % role)
        step = _grab(text, r"%s_src_step = \d \* \((.*?)\)[,;]" % role)
        # (the lane's offset for odd instructions, where the LDS layout's key changes with the instruction's parity)
        odd = re.search(r"const unsigned %s_src0_odd = \d \* \((.*)\);" % role, text)
        src0_odd = odd.group(1) if odd else src0
        edge0 = _grab(text, r"const unsigned a_edge0 = (.*), b_edge0 = .*;") if role == "a" else \
            _grab(text, r"const unsigned a_edge0 = .*, b_edge0 = (.*);")
        edge0_odd = edge_odds[role == "b"]
        if edge0_odd == role + "_edge0":
            edge0_odd = edge0
        estep = int(_grab(text, r"%s_edge0\) \+ x \* \((\d+)\) < %s_rem" % (role, "m" if role == "a" else "n")))
        for rem in (r for r in (8, 40, 120, 128, 200, 248) if r <= tile):
            rows_total = rem                     # the operand ends where the tile's valid part ends
            sizes = dict(M=rows_total, N=rows_total, K=K)
            covered = set()
            for wave in range(4):
                for lane in range(64):
                    bases = [_c_eval(e, dict(sizes, wave=wave, lane=lane)) for e in (src0, src0_odd)]
                    e0s = [_c_eval(e, dict(wave=wave, lane=lane)) for e in (edge0, edge0_odd)]
                    for it in range(tile * bk // 8 // 256):
                        if not e0s[it % 2] + it * estep < rem:
                            continue
                        off = bases[it % 2] + it * _c_eval(step, sizes)
                        # the chunk's eight elements must exist: pitch K (k-major) or rows_total
                        for e in range(8):
                            if kmajor:
                                r_, k_ = divmod(off + e, K)
                            else:
                                k_, r_ = divmod(off + e, rows_total)
                            assert 0 <= r_ < rem and 0 <= k_ < bk, (role, rem, wave, lane, it)
                            covered.add((r_, k_))
            assert covered == {(r, k) for r in range(rem) for k in range(bk)}, (role, rem)


@pytest.mark.parametrize("dtype,bk,block", [("f16", 64, 32), ("f16", 64, 16), ("e5m2", 128, 32)])
@pytest.mark.parametrize("variant", ["nn", "tt"])
def test_last_k_tile_zeroes_exactly_what_lies_past_k(dtype, bk, block, variant):
    """In the last k-tile of a ragged K the EDGE instantiation keeps a lane in instruction ``x``'s mask while
    ``k0 + x*step < klim``: the slots of the other lanes are written as zeros, once, instead of being fetched.
    For every ``klim`` in whole chunks, replay the guards
    over all slots: a slot is zeroed exactly when the chunk that the layout puts there starts at or past
    ``klim`` (chunks never straddle it), so the tile ends up holding the operand's k-values below
    ``klim`` and zeros above."""
    ta, tb = variant[0] == "t", variant[1] == "t"
    tile = 256
    unit, _ = gemm.emit(bm=tile, bn=tile, bk=bk, trans_a=ta, trans_b=tb, with_grouped=False, dtype=dtype, block=block)
    text = unit.text
    esize = 2 if dtype == "f16" else 1
    epc = 16 // esize
    K = 2 * bk
    sizes = dict(M=512, N=512, K=K)
    k0s = _grab(text, r"const unsigned a_k0 = (.*), b_k0 = .*;"), _grab(text, r"const unsigned a_k0 = .*, b_k0 = (.*);")
    for role, rows_total, kmajor, k0_text in (("a", 512, not ta, k0s[0]), ("b", 512, tb, k0s[1])):
        src0 = _grab(text, r"const unsigned %s_src0 = \d \* \((.*)\);" % role)
        step = _grab(text, r"%s_src_step = \d \* \((.*?)\)[,;]" % role)
        # (the lane's offset for odd instructions, where the LDS layout's key changes with the instruction's parity)
        odd = re.search(r"const unsigned %s_src0_odd = \d \* \((.*)\);" % role, text)
        src0_odd = odd.group(1) if odd else src0
        kstep = int(_grab(text, r"%s_k0 \+ x \* \((\d+)\) < klim_nx" % role))
        iters = tile * bk // epc // 256
        for klim in range(epc, bk + 1, epc):
            zeroed, fetched = set(), set()
            for wave in range(4):
                for lane in range(64):
                    bases = [_c_eval(e, dict(sizes, wave=wave, lane=lane)) for e in (src0, src0_odd)]
                    k0 = _c_eval(k0_text, dict(wave=wave, lane=lane))
                    for it in range(iters):
                        off = bases[it % 2] + it * _c_eval(step, sizes)
                        r_, k_ = divmod(off, K) if kmajor else divmod(off, rows_total)[::-1]
                        assert k_ == k0 + it * kstep, (role, wave, lane, it)      # the guard sees the chunk's own k
                        (zeroed if k0 + it * kstep >= klim else fetched).add((r_, k_))
            if kmajor:
                assert fetched == {(r, k) for r in range(tile) for k in range(0, klim, epc)}
            else:
                assert fetched == {(r, k) for r in range(0, tile, epc) for k in range(klim)}
            assert len(zeroed) + len(fetched) == tile * bk // epc
