"""Bank arithmetic of the XOR-rotated LDS layouts (CPU only).

LDS model, fitted to SQ_LDS_BANK_CONFLICT measurements of single-wave access patterns on
gfx950: 4-byte accesses are served 32 lanes at a time over 32 banks (``address % 32``);
8-byte accesses 32 lanes at a time and 16-byte reads 16 lanes at a time over 64 banks;
16-byte writes 8 lanes at a time.  Within a pass no two lanes may touch the same bank at
different addresses.  The GEMM layouts measure SQ_LDS_BANK_CONFLICT = 0 on the GPU.
"""
import itertools

import numpy as np
import pytest

from lego_amd.kernels import gemm, transpose
from oracle import lego_index as li


def conflicts(word_addrs, words_per_lane, write=False):
    """Worst number of distinct addresses per bank within a pass (1 = conflict free)."""
    lanes_per_pass = {1: 32, 2: 32, 4: 8 if write else 16}[words_per_lane]
    banks = 32 if words_per_lane == 1 else 64
    worst = 1
    for g in range(0, 64, lanes_per_pass):
        per_bank = {}
        for lane in range(g, g + lanes_per_pass):
            for w in range(words_per_lane):
                a = int(word_addrs[lane]) + w
                per_bank.setdefault(a % banks, set()).add(a)
        worst = max(worst, max(len(s) for s in per_bank.values()))
    return worst


@pytest.mark.parametrize("esize,tile,group", [(4, (32, 32), (1, 8)), (4, (32, 32), (2, 2)), (4, (32, 32), (2, 4)),
                                              (2, (64, 64), (1, 4)), (2, (64, 64), (1, 1))])
def test_transpose_staging_is_bijective_and_conflict_free(esize, tile, group):
    sr, sc = tile[0] * group[0], tile[1] * group[1]
    kd, vec = sc * esize // 4, 16 // esize
    rows_per_read = 4 if esize == 4 else 8
    lay = transpose.staging_layout(kd, sr, esize)
    table = np.array([[int(lay.apply(k, r)) for r in range(sr)] for k in range(kd)])
    assert sorted(table.ravel().tolist()) == list(range(kd * sr))          # a bijection of the tile
    # the closed form of the oracle's xor_swizzle family
    pack = transpose.pack_factor(sr)
    for k, r in itertools.product(range(0, kd, 7), range(0, sr, 5)):
        row, pos = k // pack, (k % pack) * sr + r
        assert table[k, r] == row * pack * sr + (pos ^ int(transpose.staging_key(k, sr, esize)))
        assert tuple(int(v) for v in lay.inv_raw(int(table[k, r]))) == (k, r)
    # 16-byte row groups stay contiguous and aligned (phase 2 reads them whole)
    for k in range(kd):
        for r0 in range(0, sr, 4):
            assert table[k, r0] % 4 == 0 and list(table[k, r0:r0 + 4]) == list(range(table[k, r0], table[k, r0] + 4))
    threads = 256
    # every vector of the macro tile is loaded exactly once
    steps = sr * sc // (vec * threads)
    seen = {tuple(int(v) for v in transpose.phase1_vector(sr, sc // vec, esize, it, t))
            for it in range(steps) for t in range(threads)}
    assert seen == set(itertools.product(range(sr), range(sc // vec)))
    # phase 1: lane t of wave w stores word e of vector (it*256 + t) -> 4-byte scattered stores
    for it in range(sr * sc // (vec * threads)):
        for wave in range(4):
            for e in range(4):
                addrs = []
                for lane in range(64):
                    r, cv = transpose.phase1_vector(sr, sc // vec, esize, it, wave * 64 + lane)
                    addrs.append(table[cv * 4 + e, r])
                assert conflicts(addrs, 1) == 1, (it, wave, e)
    # phase 2: 16-byte reads of one row group of one word-column
    for it in range(max(1, kd * (sr // rows_per_read) // threads)):
        for wave in range(4):
            for half in range(rows_per_read // 4):
                addrs = []
                for lane in range(64):
                    w = it * threads + wave * 64 + lane
                    k, rv = w // (sr // rows_per_read), w % (sr // rows_per_read)
                    addrs.append(table[k, rv * rows_per_read + 4 * half])
                assert conflicts(addrs, 4) == 1, (it, wave, half)


def test_gemm_lds_layouts_are_bijective_and_conflict_free():
    bm, bn, bk = 256, 256, 64
    a = gemm.lds_a_layout(bm, bk // 8)
    b = gemm.lds_b_layout(bk, bn)
    ta = np.array([[int(a.apply(r, c)) for c in range(bk // 8)] for r in range(bm)])
    tb = np.array([[int(b.apply(k, n)) for n in range(bn)] for k in range(bk)])
    assert sorted(ta.ravel().tolist()) == list(range(bm * bk // 8))
    assert sorted(tb.ravel().tolist()) == list(range(bk * bn))
    # global->LDS stores: lane t holds chunk (t % 8) of row (t / 8) of A, chunk (t % 32) of k-row (t / 32) of B
    for wave in range(4):
        lanes = [wave * 64 + l for l in range(64)]
        assert conflicts([4 * ta[t // 8, t % 8] for t in lanes], 4, write=True) == 1
        assert conflicts([tb[t // 32, 8 * (t % 32)] // 2 for t in lanes], 4, write=True) == 1
    # A fragments: lane l reads chunk (2*ks + l/32) of row (l % 32) -> ds_read_b128
    for ks in range(4):
        assert conflicts([4 * ta[l % 32, 2 * ks + l // 32] for l in range(64)], 4) == 1
    # B fragments: transposing 8-byte reads, lane l -> k-row ks*16 + (l/32)*8 + h*4 + (l%16)/4,
    # columns (l/16 % 2)*16 + 4*(l % 4) ..
    for ks in range(4):
        for h in range(2):
            addrs = [tb[ks * 16 + (l // 32) * 8 + h * 4 + (l % 16) // 4, ((l // 16) % 2) * 16 + 4 * (l % 4)] // 2
                     for l in range(64)]
            assert conflicts(addrs, 2) == 1


def test_gemm_lds_layout_for_16_column_blocks_is_bijective_and_conflict_free():
    """v_mfma_f32_16x16x32: a fragment's four lane groups are four k blocks of the same 16 columns, so the two groups
    of a pass read the same columns of k-rows eight apart; the layout's key tells them apart (without it the test
    below counts two addresses per bank, and the GEMM measures SQ_LDS_BANK_CONFLICT at a third of its LDS cycles)."""
    bn, bk = 256, 64
    b = gemm.lds_b_layout(bk, bn, 4, groups_by_k=True)
    tb = np.array([[int(b.apply(k, n)) for n in range(bn)] for k in range(bk)])
    assert sorted(tb.ravel().tolist()) == list(range(bk * bn))
    for wave in range(4):      # global->LDS: chunk (t % 32) of k-row (t / 32)
        lanes = [wave * 64 + l for l in range(64)]
        assert conflicts([tb[t // 32, 8 * (t % 32)] // 2 for t in lanes], 4, write=True) == 1
    plain = gemm.lds_b_layout(bk, bn, 4)
    tp = np.array([[int(plain.apply(k, n)) for n in range(bn)] for k in range(bk)])
    for ks in range(2):
        for h in range(2):
            for j in range(16):
                rows_cols = [(ks * 32 + (l // 16) * 8 + h * 4 + (l % 16) // 4, 16 * j + 4 * (l % 4)) for l in range(64)]
                assert conflicts([tb[k, n] // 2 for k, n in rows_cols], 2) == 1
                assert conflicts([tp[k, n] // 2 for k, n in rows_cols], 2) == 2


def test_gemm_lds_layouts_8bit_are_bijective_and_conflict_free():
    """One-byte operands: 128 k-values per tile, 32 per lane and MFMA."""
    bm, bn, bk = 256, 256, 128
    a = gemm.lds_a_layout(bm, bk // 16)
    b = gemm.lds_b_layout(bk, bn, 8)
    ta = np.array([[int(a.apply(r, c)) for c in range(bk // 16)] for r in range(bm)])
    tb = np.array([[int(b.apply(k, n)) for n in range(bn)] for k in range(bk)])
    assert sorted(ta.ravel().tolist()) == list(range(bm * bk // 16))
    assert sorted(tb.ravel().tolist()) == list(range(bk * bn))
    # A fragments: lane l reads chunks 4*ks + 2*(l/32) + {0, 1} of row l % 32, two ds_read_b128
    for ks in range(2):
        for c in range(2):
            assert conflicts([4 * ta[l % 32, 4 * ks + 2 * (l // 32) + c] for l in range(64)], 4) == 1
    # B fragments: transposing 8-byte reads, lane l -> k-row ks*64 + (l/32)*32 + 8*h + (l%16)/2,
    # columns (l/16 % 2)*16 + 8*(l % 2) .. +7 (byte addresses -> words)
    for ks in range(2):
        for h in range(4):
            addrs = [tb[ks * 64 + (l // 32) * 32 + 8 * h + (l % 16) // 2, ((l // 16) % 2) * 16 + 8 * (l % 2)] // 4
                     for l in range(64)]
            assert conflicts(addrs, 2) == 1


def test_oracle_xor_swizzle_matches_product_family():
    blk = li.xor_swizzle(16, 64, unit=4, every=4, span=16)   # fp32 key of a 64-row tile, 16 vectors
    seen = set()
    for r, c in itertools.product(range(16), range(64)):
        p = blk.apply((r, c))
        assert p == r * 64 + (c ^ (((r // 4) % 16) * 4))
        assert blk.inv(p) == (r, c)
        seen.add(p)
    assert len(seen) == 16 * 64
