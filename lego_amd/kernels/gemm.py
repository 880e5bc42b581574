"""Generator of the fp16 GEMM and grouped GEMM kernels.

What LEGO contributes is what it contributes to the reference's Triton kernels
(benchmarks/triton/matmul_sympy.py:37-78, grouped_gemm_sympy.py:7-24): the offsets of the
A, B and C tiles of ``OrderBy(Row(..)).TileBy([M/BM, K/BK], [BM, BK])`` and friends, and the
grouped launch order ``OrderBy(Col(max(npm//GM,1),1), Col(min(npm,GM),npn)).TileBy([npm,npn]).inv(pid)``.
Here the same algebra also lays out what Triton hides: the lane-to-chunk assignment of
the global loads, the XOR-rotated LDS tiles (``GenP`` blocks), the MFMA operand
fragments, the accumulator-to-C map and the remap of workgroup ids onto the eight XCDs.

The grouped kernel runs one workgroup per tile of every problem; a workgroup finds its
problem from running tile totals passed as kernel arguments (the reference's kernel
scans the same totals on the device, triton_generated/grouped_gemm/grouped_gemm.py:61-82)
and then applies the grouped launch order inside that problem.
"""
from __future__ import annotations

import sympy as sp

from ..lego import BitXor, Col, GenP, OrderBy, Row
from .common import BANNER, Emitted, code, idx, size, template, tidy

XCDS = 8
CUS = 256      # MI355X: 8 XCDs of 32 CUs
MAX_GROUPS = 64
STAMP_ROWS = 8192      # workgroups whose time stamps a measurement build keeps


def lds_a_layout(bm, chunks):
    """A tile in 16-byte chunks: ``row*chunks + (chunk ^ ((row // (16/chunks)) % chunks))``.

    Sixteen lanes that read the same chunk of sixteen consecutive rows (one quarter of a
    ds_read_b128) land on sixteen different 16-byte slots of the 256-byte bank window:
    ``16/chunks`` consecutive rows fill the window once, and the key steps with every refill."""
    assert 16 % chunks == 0

    def key(row):
        return (row // (16 // chunks)) % chunks

    def forward(rc):
        row, ch = rc
        return row * chunks + BitXor(sp.sympify(ch), sp.sympify(key(row)))

    def backward(flat):
        row, p = flat // chunks, flat % chunks
        return (row, BitXor(sp.sympify(p), sp.sympify(key(row))))

    return OrderBy(GenP((bm, chunks), forward, backward)).TileBy([bm, chunks])


def lds_b_layout(bk, bn, period=4, groups_by_k=False):
    """B tile in elements, rows of ``bn``: ``k*bn + (n ^ 32*(k % period))``.

    A transposing read of 2-byte elements touches four consecutive k-rows, 64 bytes of each;
    rotating the 64-byte chunk index by ``k % 4`` puts the four rows on four different quarters
    of the banks.  One of 1-byte elements touches eight k-rows, 32 bytes of each (32 elements
    again): ``period = 8``.  Bits 0-4 of ``n`` are untouched, so 16-byte stores and 8-byte reads
    stay whole.  ``groups_by_k`` (16 x 16 MFMA blocks, 2-byte elements): the two 16-lane groups that an 8-byte read
    serves together read the same 16 columns of k-rows eight apart, 32 of the 64 bytes of each quarter; the key
    also flips bit 4 of ``n`` (32 bytes) with bit 3 of ``k``, which sends the second group to the other 32 bytes
    (bits 0-3 stay, so 16-byte stores and 8-byte reads are still whole)."""
    assert not groups_by_k or period == 4

    def key(k):
        return (k % period) * 32 + (((k // 8) % 2) * 16 if groups_by_k else 0)

    def forward(kn):
        k, n = kn
        return k * bn + BitXor(sp.sympify(n), sp.sympify(key(k)))

    def backward(flat):
        k, p = flat // bn, flat % bn
        return (k, BitXor(sp.sympify(p), sp.sympify(key(k))))

    return OrderBy(GenP((bk, bn), forward, backward)).TileBy([bk, bn])


def lds_c_layout(rows, cols, block=32):
    """A wave's block of C as fp16 in 8-byte chunks: ``row*(cols/4) + (chunk ^ key(row))``.

    32 x 32 accumulator blocks: 32 lanes store the same chunk of 32 consecutive rows; ``key = row % span``,
    ``span = min(32, cols/4)``, spreads them over 32 different chunks of the 256-byte bank window (over 16, two rows
    each, when a row has only 16 chunks).  16 x 16 blocks: the 32 lanes that are served together store two
    neighbouring chunks of 16 consecutive rows; ``key = 2*(row % 16)`` spreads the rows over the 16 chunk pairs and
    leaves a pair together and in order, so a 16-byte read-back needs no swap."""
    chunks = cols // 4
    span = min(32, chunks)

    def key(row):
        return row % span if block == 32 else 2 * (row % min(16, chunks // 2))

    def forward(rc):
        row, ch = rc
        return row * chunks + BitXor(sp.sympify(ch), sp.sympify(key(row)))

    def backward(flat):
        row, p = flat // chunks, flat % chunks
        return (row, BitXor(sp.sympify(p), sp.sympify(key(row))))

    return OrderBy(GenP((rows, chunks), forward, backward)).TileBy([rows, chunks])


def launch_order(num_pid_m, num_pid_n, group_m, pid):
    """``(pid_m, pid_n)`` of the grouped launch order (matmul_sympy.py:57-65)."""
    lay = OrderBy(Col(sp.Max(num_pid_m // group_m, 1), 1),
                  Col(sp.Min(num_pid_m, group_m), num_pid_n)).TileBy([num_pid_m, num_pid_n])
    return lay.inv(pid)


def xcd_remap(per, wg, xcds=XCDS):
    """Workgroup id -> position in the launch order such that the ids one XCD receives
    (``wg % xcds`` is constant) form a contiguous run of ``per`` positions: read ``wg`` as
    ``(j, x)`` of a row-major ``[per, xcds]`` box and store it column-major."""
    j, x = OrderBy(Row(per, xcds)).TileBy([per, xcds]).inv(wg)
    return OrderBy(Col(per, xcds)).TileBy([per, xcds])[j, x]


def lane_and_unit(expr, unit_vars, units, lane_vars, lane_values, stride):
    """Split an LDS offset ``expr`` (unit indices known at generation time, lane indices at run time) into a lane
    term and two constants per unit: ``expr(u, lane) == add[u] + (lane_term(lane) ^ xor[u])``.

    The XOR-rotated staging layouts have this shape: a unit moves the lane's offset by whole rows (a multiple of
    ``stride``: an immediate of the LDS instruction) and flips bits of the chunk index inside a row (one v_xor with
    a literal), so a lane needs one register and one instruction per access where the printed expression costs
    four or five.  Returns ``(lane_term, {unit: (add, xor)})`` after checking the identity for every unit and every
    combination of ``lane_values``; raises if the layout does not split this way."""
    xor_eval = {"BitXor": lambda a, b: int(a) ^ int(b)}
    lane_term = expr.subs({v: 0 for v in unit_vars})
    f_lane = sp.lambdify(lane_vars, lane_term, [xor_eval, "math"])
    f_full = sp.lambdify(list(unit_vars) + list(lane_vars), expr, [xor_eval, "math"])
    table = {}
    for u in units:
        add = xor = None
        for lv in lane_values:
            full, base = int(f_full(*u, *lv)), int(f_lane(*lv))
            if not 0 <= base < stride:
                raise ValueError("the lane term leaves the first stride")
            a, x = full // stride * stride, (full % stride) ^ base
            if add is None:
                add, xor = a, x
            elif (a, x) != (add, xor):
                raise ValueError(f"offset of unit {u} is not stride*n + (lane ^ constant)")
        table[tuple(u)] = (add, xor)
    return lane_term, table


LAST_KTILE_RING = 8      # vectors a lane holds between reading them back from the staging block and storing them


def last_ktile_schedule(TM, TN, NPH, WN, block=32, mps=1):
    """Slot schedule of a tile's last k-tile, in which the result leaves under the MFMAs.

    ``TM x TN`` accumulator blocks of ``block x block`` per wave, ``NPH`` k-steps per k-tile, ``mps`` MFMAs per slot (a
    slot is what one scheduling fence encloses: 32 cycles of MFMA, so one 32x32x16 or two 16x16x32).  The MFMAs go
    block row by block row (``i``), within a row k-step by k-step (MFMA ``i*TN*NPH + ks*TN + j``), so the accumulators
    of block row ``i`` are final when row ``i+1`` starts.  A slot also carries
      loads   during row 0, every operand fragment the k-tile still needs, in the order of their first use (the
              first slots carry one more than the rest): after row 0 no wave reads the operand buffers any more, and
              a barrier there hands all of LDS to the staging of the results;
      stage   during row ``i+1``, block row ``i`` converted and written to the wave's staging block, a unit =
              four columns of a lane = (block, q), spread evenly over the row's slots;
      rb, st  during row ``i+2``, the staged rows of block row ``i`` read back as 16-byte vectors (``rb``) and
              stored to C two slots later (``st``: the LDS latency passes under the MFMAs between).
    What falls past the last row -- the staging of the last block row, the stores of the last two -- is the
    ``tail``, in the same order without MFMAs.  With more than one MFMA per slot the MFMAs are inline assembly whose
    wait states the compiler does not know: the tail then holds a ``fence`` (a scheduling fence and the wait states
    of the longest MFMA) in front of the first unit whose block took its last MFMA in the very last slot, so that
    the read of that result cannot be issued too close behind it.  Returns ``(slots, tail)``; a slot is a dict with the keys
    ``mfmas`` [(i, j, ks)], ``loads`` [(ks, f)], ``stage`` [(i, j, q)], ``rb`` [it], ``st`` [it], ``barrier``."""
    Q = block * block // 64 // 4       # units of four accumulator registers per block
    assert TN * NPH % mps == 0 and block * WN % 512 == 0
    SPR, IPR = TN * NPH // mps, block * WN // 512      # slots, and read-backs (64 lanes x 16 bytes), per block row
    G = TM * SPR
    slots = [dict(mfmas=[], loads=[], stage=[], rb=[], st=[], barrier=False) for _ in range(G)]
    for i in range(TM):
        for ks in range(NPH):
            for j in range(TN):
                slots[(i * TN * NPH + ks * TN + j) // mps]["mfmas"].append((i, j, ks))
    need = []                      # (ks, f): f < TM a fragment of A's block row f, else of B's block column f - TM
    for ks in range(1, NPH):
        need += [(ks, 0)] + [(ks, TM + j) for j in range(TN)]
    for i in range(1, TM):
        need += [(ks, i) for ks in range(1, NPH)]
    at = 0
    for s_ in range(SPR):      # spread over the slots of row 0, the first slots one more than the rest
        for _ in range(len(need) // SPR + (1 if s_ < len(need) % SPR else 0)):
            slots[s_]["loads"].append(need[at])
            at += 1
    assert at == len(need)
    slots[SPR - 1]["barrier"] = True
    late = []                      # (global slot, order, kind, payload) of what falls past the last MFMA
    def put(g, kind, payload):
        if g < G:
            slots[g][kind].append(payload)
        else:
            late.append((g, len(late), kind, payload))
    for r in range(TM):
        for u, (j, q) in enumerate((j, q) for j in range(TN) for q in range(Q)):
            put((r + 1) * SPR + u * SPR // (TN * Q), "stage", (r, j, q))
        for m in range(IPR):
            g = (r + 2) * SPR + m * SPR // IPR
            put(g, "rb", r * IPR + m)
            put(g + 2, "st", r * IPR + m)
    # Past the last MFMA nothing hides a latency, so the order is by dependence: the stores whose vectors are already
    # on their way, then the read-backs of rows staged earlier (up to RING vectors in flight) with the staging of the
    # last block row behind them, their stores, and the last block row in batches of RING.
    ordered = [(kind, payload) for _, _, kind, payload in sorted(late)]
    in_slots = {it for slot in slots for it in slot["rb"]}
    tail = [(kind, it) for kind, it in ordered if kind == "st" and it in in_slots]
    early = [it for kind, it in ordered if kind == "rb" and it // IPR < TM - 1]
    assert len(early) <= LAST_KTILE_RING
    tail += [("rb", it) for it in early]
    fenced = False
    for kind, u in ordered:
        if kind == "stage":
            if mps > 1 and not fenced and (u[0] * TN * NPH + (NPH - 1) * TN + u[1]) // mps == G - 1:
                tail.append(("fence", None))
                fenced = True
            tail.append((kind, u))
    tail += [("st", it) for it in early]
    fresh = [it for kind, it in ordered if kind == "rb" and it // IPR == TM - 1]
    for first in range(0, len(fresh), LAST_KTILE_RING):
        batch = fresh[first:first + LAST_KTILE_RING]
        tail += [("rb", it) for it in batch] + [("st", it) for it in batch]
    return slots, tail


def _tile_params(bm, bn, bk, waves, max_group_m, trans_a, trans_b, with_grouped, dtype, block=32, suffix="", stamps=False):
    """Everything the templates need for one tile shape.  ``block``: 32 = v_mfma_f32_32x32x16 (x64 for 8-bit operands),
    16 = v_mfma_f32_16x16x32 (16-bit operands), the side of an accumulator block."""
    # element type, bytes per element, k-depth of one MFMA, result type; the 8-bit types are the
    # OCP formats of v_mfma_f32_32x32x64_f8f6f4 (format code 0 = e4m3, 1 = e5m2)
    # "bf16h": bfloat16 operands with the fp16 result that the reference's matmul stores whatever its
    # operands' 16-bit type (matmul_sympy.py:129-145, 203)
    elt, esize, mfma_k, out_elt = {"f16": ("_Float16", 2, 16, "_Float16"), "bf16": ("__bf16", 2, 16, "__bf16"),
                                   "bf16h": ("__bf16", 2, 16, "_Float16"),
                                   "e4m3": ("unsigned char", 1, 64, "_Float16"),
                                   "e5m2": ("unsigned char", 1, 64, "_Float16")}[dtype]
    EPC = 16 // esize                      # elements per 16-byte chunk
    assert not (with_grouped and dtype != "f16"), "the grouped kernel is built for fp16 only"
    assert block in (32, 16) and (block == 32 or esize == 2)
    if block == 16:
        mfma_k = 32
    MPS = 32 // block                      # MFMAs per scheduling slot: a slot is 32 cycles of matrix-core work
    WAVES_M, WAVES_N = waves
    THREADS = 64 * WAVES_M * WAVES_N
    WM, WN = bm // WAVES_M, bn // WAVES_N
    TM, TN = WM // block, WN // block
    A_ITERS = bm * bk // EPC // THREADS
    B_ITERS = bk * bn // EPC // THREADS
    assert bm * bk // EPC % THREADS == 0 and bk * bn // EPC % THREADS == 0 and bk % mfma_k == 0
    NPH = bk // mfma_k                     # MFMA phases per k-tile
    assert WN >= 64 and WN % 32 == 0
    # Slot schedule of the main loop.  A phase has TM*TN MFMA slots; the TM+TN fragment loads of the
    # next phase and the memory->LDS instructions are spread evenly over them (for the 256x256
    # tile: a fragment on every even slot, a copy on every odd one).  The copies of a k-tile go into
    # the phase after the barrier (the first DMA_LAST) and the phase that follows it (the rest).
    SLOTS, FRAGS, COPIES = TM * TN // MPS, TM + TN, A_ITERS + B_ITERS
    assert NPH >= 2 and NPH % 2 == 0, "fragments are double buffered by phase parity"
    # With two phases per k-tile (8-bit operands) the phase before the barrier is the only one a copy issued in it
    # would have to land in: all copies go behind the barrier, one per slot, and have the whole next phase
    # (8192^3 e5m2: 2.75 -> 2.92 PFLOP/s).  With four phases the split 8 + 8 measures best (all 16 behind the barrier,
    # on top of a fragment load in every other slot, overfill the slots: -4 % on fp16).
    DMA_LAST = min(COPIES, SLOTS if NPH == 2 else SLOTS // 2 if SLOTS >= 2 * FRAGS else SLOTS)
    assert COPIES - DMA_LAST <= SLOTS

    def spread(first, count):
        """``count`` items ``first, first+1, ...`` on slots ``floor((q + 1/2) * SLOTS / count)``."""
        out = [[] for _ in range(SLOTS)]
        for q in range(count):
            out[(2 * q + 1) * SLOTS // (2 * count)].append(first + q)
        return out

    load_slots = [[] for _ in range(SLOTS)]
    for f in range(FRAGS):
        load_slots[f * SLOTS // FRAGS].append(f)
    dma_last, dma_first = spread(0, DMA_LAST), spread(DMA_LAST, COPIES - DMA_LAST)
    none = [[] for _ in range(SLOTS)]
    last_slots, last_tail = last_ktile_schedule(TM, TN, NPH, WN, block, MPS)

    M, N, K = size("M"), size("N"), size("K")
    npm, npn, per_xcd, group_m = size("num_pid_m"), size("num_pid_n"), size("wg_per_xcd"), size("GM")
    t, it, wave, wg, pid, k, ks = (idx(n) for n in ("t", "it", "wave", "wg", "pid", "k", "ks"))
    pid_m, pid_n = idx("pid_m"), idx("pid_n")
    row, ch, kr = idx("row"), idx("ch"), idx("kr")
    i, j, r, q = idx("i"), idx("j"), idx("r"), idx("q")
    wm, wn, l32, lhi, l16, lgrp = (idx(n) for n in ("wm", "wn", "l32", "lhi", "l16", "lgrp"))
    cr, cc = idx("cr"), idx("cc")

    # the reference's operand layouts with its transpose flags (matmul_sympy.py:37-46): a transposed
    # operand is the column-major layout of the same logical matrix
    A_L = OrderBy(Col(M, K) if trans_a else Row(M, K)).TileBy([M / bm, K / bk], [bm, bk])
    B_L = OrderBy(Col(K, N) if trans_b else Row(K, N)).TileBy([K / bk, N / bn], [bk, bn])
    C_L = OrderBy(Row(M, N)).TileBy([M / bm, N / bn], [bm, bn])
    # An operand tile is "k-major" when its k-values are contiguous in memory (A as given, B
    # transposed): it is staged as [row][16-byte chunk of k] and a fragment is one 16-byte read.
    # Otherwise (B as given, A transposed) it is staged as in memory, [k][row], and a fragment is
    # two transposing 8-byte reads.
    a_kmajor, b_kmajor = not trans_a, trans_b

    wm_e, wn_e = OrderBy(Row(WAVES_M, WAVES_N)).TileBy([WAVES_M, WAVES_N]).inv(wave)

    rng = {row: (0, bm), ch: (0, bk // EPC), kr: (0, bk), i: (0, TM), j: (0, TN), r: (0, 16),
           wm: (0, WAVES_M), wn: (0, WAVES_N), l32: (0, 32), lhi: (0, 2), l16: (0, 16),
           lgrp: (0, 4), ks: (0, NPH), cr: (0, bm), cc: (0, bn), pid_m: (0, M / bm),
           pid_n: (0, N / bn), k: (0, K / bk)}
    # the lane's row (column) of an MFMA operand block and its k block: lane % 32 and lane / 32 for 32 x 32 blocks,
    # lane % 16 and lane / 16 for 16 x 16 ones
    lrow, lk = (l32, lhi) if block == 32 else (l16, lgrp)

    def chunk_walk(expr, n_iters):
        """``expr`` (a function of the lane ``t`` and the chunk counter ``it``) as ``base[it % 2] + it*step`` with a
        lane-independent ``step``: ``(base[0], base[1], step)``, the two bases equal when the walk is affine (they
        differ where the LDS layout's key changes with the parity of the instruction); raises if it is neither."""
        lane_s, rng_l = idx("lane"), {idx("lane"): (0, 64), wave: (0, WAVES_M * WAVES_N)}
        at = [tidy(sp.sympify(expr).subs(it, v), rng_l) for v in range(n_iters)]
        two = sp.simplify(at[2] - at[0]) if n_iters > 2 else sp.simplify(2 * (at[1] - at[0])) if n_iters > 1 else sp.Integer(0)
        if two.free_symbols & {lane_s, wave}:
            # not visibly uniform: decide by exhaustive evaluation below
            two = sp.simplify(two.subs({lane_s: 0, wave: 0}))
        step = sp.simplify(two / 2)
        base = [at[0], tidy(at[1] - step, rng_l) if n_iters > 1 else at[0]]
        names = sorted(set().union(*(e.free_symbols for e in at + [step])) - {lane_s, wave}, key=str)
        sizes = {s_: 8192 + 256 * n_ for n_, s_ in enumerate(names)}
        evaluate = [{"BitXor": lambda a_, b_: int(a_) ^ int(b_)}, "math"]
        same = True
        for v in range(n_iters):   # exhaustive over lanes and waves
            diff = sp.lambdify([lane_s, wave], (at[v] - base[v % 2] - v * step).subs(sizes), evaluate)
            gap = sp.lambdify([lane_s, wave], (base[1] - base[0]).subs(sizes), evaluate)
            for w_ in range(WAVES_M * WAVES_N):
                for l_ in range(64):
                    if diff(l_, w_) != 0:
                        raise ValueError("chunk offsets are not affine in the instruction counter, by parity either")
                    same = same and gap(l_, w_) == 0
        return base[0], (base[0] if same else base[1]), step

    Cs_L = lds_c_layout(WM, WN, block)
    cp = idx("cp")
    rng.update({cr: (0, WM), cp: (0, WN // 8)})
    lane_o = idx("lane")
    c_out = [tidy(e, {lane_o: (0, 64), it: (0, WM * WN // 8 // 64)}) for e in
             OrderBy(Row(WM, WN // 8)).TileBy([WM, WN // 8]).inv(it * 64 + lane_o)]

    pm_e, pn_e = launch_order(npm, npn, group_m, pid)

    # The staging block of the results, as the last k-tile's schedule addresses it (elements of the result type):
    # a unit (i, j, q) writes four columns of a lane, a read-back `it` fetches 16 bytes of row 4*it + lane/16.
    # (a lane of a 32 x 32 block holds columns 8q + 4*(lane/32) .. +3 of row lane%32 in registers 4q..4q+3, a lane of a
    # 16 x 16 block columns 4*(lane/16) .. +3 of row lane%16 in its four registers)
    if block == 32:
        stage_e = tidy(4 * Cs_L[i * 32 + l32, j * 8 + q * 2 + lhi], rng)
        back_e = (tidy(4 * Cs_L[cr, 2 * cp], rng) - 4 * (cr % 2)).subs({cr: c_out[0], cp: c_out[1]})
    else:
        stage_e = tidy(4 * Cs_L[i * 16 + l16, j * 4 + lgrp], rng) + 0 * q
        back_e = tidy(4 * Cs_L[cr, 2 * cp], rng).subs({cr: c_out[0], cp: c_out[1]})     # pairs stay in order: no swap
    lanes_mfma = [(a_, b_) for a_ in range(block) for b_ in range(64 // block)]
    stage_lane, stage_ax = lane_and_unit(stage_e, (i, j, q), [(a_, b_, c_) for a_ in range(TM) for b_ in range(TN) for c_ in range(block * block // 256)],
                                         (lrow, lk), lanes_mfma, block * WN)
    n_its = WM * WN // 8 // 64
    back_lane, back_ax = lane_and_unit(back_e, (it,), [(a_,) for a_ in range(n_its)], (lane_o,), [(a_,) for a_ in range(64)], 512)      # a wave instruction moves 64 x 8 elements

    def with_constants(kind, payload):
        if kind == "stage":
            return tuple(payload) + stage_ax[tuple(payload)]
        return (payload,) + back_ax[(payload,)] if kind == "rb" else payload      # "st": the vector, "fence": nothing
    for slot_ in last_slots:
        slot_["stage"] = [with_constants("stage", u) for u in slot_["stage"]]
        slot_["rb"] = [with_constants("rb", u) for u in slot_["rb"]]
    last_tail = [(kind, with_constants(kind, u)) for kind, u in last_tail]
    # C: the wave's first row and column are uniform, a lane adds its row and 16-byte column, a read-back four rows
    c_full_e = tidy(C_L[pid_m, pid_n, wm * WM + cr, wn * WN + 8 * cp], rng).subs({cr: c_out[0], cp: c_out[1]})
    c_wave_e = c_full_e.subs({it: 0, lane_o: 0})
    c_lane_e = c_full_e.subs({pid_m: 0, pid_n: 0, wm: 0, wn: 0, it: 0})
    c_it_e = sp.expand(c_full_e.subs(it, 1) - c_full_e.subs(it, 0))
    assert sp.expand(c_full_e - (c_wave_e + c_lane_e + it * c_it_e)) == 0, "C offsets are not wave + lane + it*step"

    # memory->LDS: instruction `it` of wave `wave` fills slots (it*WAVES + wave)*64 + lane; the chunk
    # that lives in a slot is the inverse of the LDS layout
    WAVES = WAVES_M * WAVES_N
    lane_s = idx("lane")
    slot = (it * WAVES + wave) * 64 + lane_s
    slot_rng = {lane_s: (0, 64), wave: (0, WAVES), it: (0, max(A_ITERS, B_ITERS))}

    def operand(role):
        """Everything the template needs for operand ``role``: where a lane's memory->LDS chunk
        comes from, the k-tile stride, and the text that reads one MFMA fragment."""
        kmajor = a_kmajor if role == "a" else b_kmajor
        rows, tile_id = (bm, pid_m) if role == "a" else (bn, pid_n)
        wave_off, sub = (wm * WM + i * block, i) if role == "a" else (wn * WN + j * block, j)
        n_iters = A_ITERS if role == "a" else B_ITERS

        def glob(row_e, kk_e):   # offset of element (row, kk) of k-tile k of this operand's tile
            return A_L[pid_m, k, row_e, kk_e] if role == "a" else B_L[k, pid_n, kk_e, row_e]

        if kmajor:
            lds = lds_a_layout(rows, bk // EPC)
            r_e, ch_e = (tidy(e, slot_rng) for e in lds.inv(slot))
            full = tidy(glob(row, ch * EPC), rng)
            placed = full.subs({row: r_e, ch: ch_e})
            # a lane's k-values of its row of the block (mfma_k/2 of them for 32-row blocks, mfma_k/4 for 16-row ones): one
            # 16-byte chunk (2-byte elements) or two
            k_blocks = 64 // block
            n_ch = mfma_k // k_blocks // EPC
            chunks = [code(tidy(EPC * lds[wave_off + lrow, (ks * k_blocks + lk) * n_ch + c], rng)) for c in range(n_ch)]
            if esize == 2:
                frag = "*reinterpret_cast<const half8*>(%ss + (%s))" % (role, chunks[0])
            else:
                frag = "read_k_fragment(%s)" % ", ".join("%ss + (%s)" % (role, c) for c in chunks)
        else:
            lds = lds_b_layout(bk, rows, 4 if esize == 2 else 8, groups_by_k=block == 16)
            kr_e, col_e = (tidy(e, slot_rng) for e in lds.inv(EPC * slot))
            full = tidy(glob(EPC * ch, kr), rng)    # here `ch` counts 16-byte chunks along the row
            placed = full.subs({kr: kr_e, ch: tidy(col_e / EPC, slot_rng)})
            if esize == 2 and block == 16:
                # (16-column blocks: the four lane groups are the four k blocks of eight)
                frag_k = [ks * 32 + lgrp * 8 + h * 4 + l16 // 4 for h in (0, 1)]
                frag_c = wave_off + 4 * (l16 % 4)
            elif esize == 2:
                # a transposing read hands lane 16g+i four consecutive k of column i of group g's
                # 16 columns; source lane s supplies k-row s/4 and columns 4*(s%4)..+3
                frag_k = [ks * 16 + (lgrp // 2) * 8 + h * 4 + l16 // 4 for h in (0, 1)]
                frag_c = wave_off + (lgrp % 2) * 16 + 4 * (l16 % 4)
            else:
                # 8-bit: eight consecutive k per read; source lane s supplies k-row s/2 and columns
                # 8*(s%2)..+7 (even source lanes feed lanes 0-7 of the group, odd ones lanes 8-15)
                frag_k = [ks * 64 + (lgrp // 2) * 32 + h * 8 + l16 // 2 for h in range(4)]
                frag_c = wave_off + (lgrp % 2) * 16 + 8 * (l16 % 2)
            frag = ("read_t_fragment(%s)"
                    % ", ".join("%ss + (%s)" % (role, code(tidy(lds[fk, frag_c], rng))) for fk in frag_k))
        src0, src1, step = chunk_walk(placed.subs({tile_id: 0, k: 0}), n_iters)
        # what bounds a chunk at a ragged edge: its row of the tile (k-major: the row changes with the
        # instruction) or its first column (the other kind: the same for every instruction, or one of two by
        # the instruction's parity)
        edge0, edge1, edge_step = chunk_walk(r_e if kmajor else col_e, n_iters)
        assert kmajor or edge_step == 0
        # the first k-value (within the tile) of a lane's chunk: what a ragged last k-tile is masked by
        kedge0, kedge1, kedge_step = chunk_walk(EPC * ch_e if kmajor else kr_e, n_iters)
        assert kedge1 is kedge0
        return {f"{role}_src0": code(src0), f"{role}_src_step": code(step),
                f"{role}_src0_odd": None if src1 is src0 else code(src1),
                f"{role}_edge0": code(edge0), f"{role}_edge_step": code(edge_step),
                f"{role}_edge0_odd": None if edge1 is edge0 else code(edge1),
                f"{role}_kedge0": code(kedge0), f"{role}_kedge_step": code(kedge_step),
                f"{role}_goff_base": code(full.subs({k: 0, row: 0, ch: 0, kr: 0})),
                f"{role}_kstep": code(sp.simplify(full.subs(k, k + 1) - full)),
                f"{role}_frag_code": frag}

    variant = ("t" if trans_a else "n") + ("t" if trans_b else "n")
    tag = ("" if (bm, bn) == (256, 256) else f"_t{bm}x{bn}") + ("" if tuple(waves) == (2, 2) else f"_w{WAVES_M}x{WAVES_N}") + suffix
    chunk_params = dict(WAVES=WAVES, variant=variant, tag=tag, with_grouped=with_grouped, **operand("a"), **operand("b"))

    params = dict(
        banner=BANNER, elt=elt, out_elt=out_elt, ESIZE=esize, EPC=EPC, MFMA_K=mfma_k, NPH=NPH,
        FMT={"e4m3": 0, "e5m2": 1}.get(dtype, 0), dt=dtype, mfma_dt={"bf16h": "bf16"}.get(dtype, dtype), BM=bm, BN=bn, BK=bk, THREADS=THREADS, WAVES_M=WAVES_M, WAVES_N=WAVES_N,
        WM=WM, WN=WN, TM=TM, TN=TN, A_ITERS=A_ITERS, B_ITERS=B_ITERS, DMA_LAST=DMA_LAST,
        # s_waitcnt immediate: vmcnt in bits 3:0 and 15:14, expcnt and lgkmcnt left at their maxima
        WAIT_DMA_LAST="0x%04X" % (0x0F70 | (DMA_LAST % 16) | ((DMA_LAST // 16) << 14)),
        load_slots=load_slots, dma_last=dma_last, dma_first=dma_first, dma_none=none, XCDS=XCDS, MAX_GROUPS=MAX_GROUPS,
        last_slots=last_slots, last_tail=last_tail, RING=LAST_KTILE_RING,
        pid_layout="OrderBy(Col(max(npm//GM,1),1), Col(min(npm,GM),npn)).TileBy([npm,npn]).inv(pid)",
        MAX_GM=max_group_m,
        xcd_layout=f"OrderBy(Col(nwg/{XCDS}, {XCDS})).TileBy([nwg/{XCDS}, {XCDS}])[Row(nwg/{XCDS}, {XCDS}).inv(wg)]",
        a_layout=f"OrderBy({'Col' if trans_a else 'Row'}(M,K)).TileBy([M/{bm},K/{bk}],[{bm},{bk}])",
        b_layout=f"OrderBy({'Col' if trans_b else 'Row'}(K,N)).TileBy([K/{bk},N/{bn}],[{bk},{bn}])",
        a_kmajor=a_kmajor, b_kmajor=b_kmajor,
        c_layout=f"OrderBy(Row(M,N)).TileBy([M/{bm},N/{bn}],[{bm},{bn}])",
        wm=code(wm_e), wn=code(wn_e),
        # offset of a chunk = tile base (uniform) + position inside k-tile 0 (per lane) + k * step
        **chunk_params,
        # accumulator -> staging: row i*32 + l32, 8-byte chunk (j*32 + q*8 + lhi*4)/4 of the wave's block
        c_stage_store=code(stage_e),
        # staging -> memory: lane reads the pair of chunks (2p, 2p+1) of row cr; the XOR keeps a
        # pair together and (32 x 32 blocks) swaps its halves on odd rows
        c_out_row=code(c_out[0]), c_out_pair=code(c_out[1]),
        c_stage_load=code(tidy(4 * Cs_L[cr, 2 * cp], rng) - (4 * (cr % 2) if block == 32 else 0)),
        BLOCK=block, MPS=MPS, ACC_REGS=block * block // 64, SWAP_ODD_ROWS=block == 32, STAMPS=stamps, STAMP_ROWS=STAMP_ROWS,
        c_goff=code(tidy(C_L[pid_m, pid_n, wm * WM + cr, wn * WN + 8 * cp], rng)),
        c_stage_lane=code(stage_lane), c_back_lane=code(back_lane),
        c_wave=code(c_wave_e), c_lane=code(c_lane_e), c_it_step=code(c_it_e),
        c_lane_row=code(c_out[0].subs(it, 0)), c_lane_pair=code(c_out[1].subs(it, 0)), C_ROWS_PER_IT=64 // (WN // 8),
        # the four columns that registers 4q..4q+3 of a lane hold of block (i, j): row and first column within the tile
        c_goff_reg=code(tidy(C_L[pid_m, pid_n, idx("row"), idx("col")], {**rng, idx("row"): (0, bm), idx("col"): (0, bn)})),
        xcd_pid=code(tidy(xcd_remap(per_xcd, wg), {wg: (0, per_xcd * XCDS)})), CUS=CUS,
        pid_m=code(pm_e), pid_n=code(pn_e),
    )
    return params


def class_order(p, count, first_wg, cus=CUS, xcds=XCDS):
    """Place, among ``count`` tiles of equal depth, of the workgroup that is number ``p`` of those working on
    them (``first_wg``: the id of number 0), with integers, as the grouped kernels compute it: rounds of
    ``cus`` workgroups in order, and within a round ``xcd_remap`` over the round's length when ids and XCDs
    line up (``first_wg`` and the length multiples of ``xcds``)."""
    wg = p % cus
    round0 = p - wg
    length = cus if round0 + cus <= count else count - round0
    if first_wg % xcds or length % xcds:
        return p
    return round0 + int(xcd_remap(length // xcds, wg))


def split_order(split, wg):
    """``(tile, half)`` of workgroup ``wg`` among the ``2*split`` workgroups that share ``split``
    tiles between two halves each: ``Row(split, 2).inv(wg)``."""
    return OrderBy(Row(split, 2)).TileBy([split, 2]).inv(wg)


def emit(bm=256, bn=256, bk=64, waves=(2, 2), max_group_m=8, trans_a=False, trans_b=False, with_grouped=True,
         dtype="f16", with_split=False, with_splitk=False, block=32, suffix="", stamps=False):
    """One translation unit: the GEMM kernel of one operand layout and element type on ``bm x bn``
    tiles, with ``with_grouped`` the grouped kernel on the same tiles, and with ``with_split`` a
    second grouped kernel that gives the last tiles of its launch to two workgroups each, as
    halves of ``bm/2 x bn`` (the tail of a launch whose last round of whole tiles would leave most
    CUs idle).  ``block``: the side of the MFMA's accumulator block (see ``_tile_params``); ``suffix`` goes behind
    the names of the file and the launchers (a second build of one shape); ``stamps``: a measurement build whose
    workgroups record the real-time counter at fixed points of their tile (``lego_gemm_stamps_read``)."""
    assert not (with_splitk and block != 32), "partial sums along K are laid out for 32 x 32 accumulator blocks"
    params = _tile_params(bm, bn, bk, waves, max_group_m, trans_a, trans_b, with_grouped, dtype, block, suffix, stamps)
    ns = f"t{bm}x{bn}"
    tiles = [dict(ns=ns, text=template("gemm_tile.hip.j2").render(**params))]
    params.update(main_ns=ns, with_split=with_split, with_splitk=with_splitk)
    if with_split:
        assert with_grouped
        half = _tile_params(bm // 2, bn, bk, waves, max_group_m, trans_a, trans_b, True, dtype, block, stamps=stamps)
        hns = f"t{bm // 2}x{bn}"
        tiles.append(dict(ns=hns, text=template("gemm_tile.hip.j2").render(**half)))
        split, swg, ti, hf = size("split"), idx("swg"), idx("pid_m"), idx("half")
        tile_e, half_e = (tidy(e, {swg: (0, 2 * split)}) for e in split_order(split, swg))
        params.update(half_ns=hns, HBM=bm // 2,
                      split_layout="OrderBy(Row(split, 2)).TileBy([split, 2]).inv(s)",
                      split_tile=code(tile_e), split_half=code(half_e),
                      # rows of halves in place of rows of tiles: one more level under the tile row
                      half_pid_m=code(tidy(OrderBy(Row(size("num_pid_m"), 2)).TileBy([size("num_pid_m"), 2])[ti, hf],
                                           {ti: (0, size("num_pid_m")), hf: (0, 2)})))
    params["tiles"] = tiles
    text = template("gemm.hip.j2").render(**params)
    variant, tag = params["variant"], params["tag"]
    meta = dict(BM=bm, BN=bn, BK=bk, MAX_GROUPS=MAX_GROUPS)
    launchers = [f"lego_gemm_{dtype}_{variant}{tag}_launch"] + ([f"lego_grouped_gemm_f16{tag}_launch"] if with_grouped else [])
    if with_split:
        launchers.append(f"lego_grouped_gemm_f16{tag}_split_launch")
    if with_splitk:
        launchers.append(f"lego_gemm_{dtype}_{variant}{tag}_splitk_launch")
    if stamps:
        launchers.append("lego_gemm_stamps_read")
    return Emitted(f"gemm_{dtype}_{variant}{tag}.hip", text, launchers), meta


def emit_any(bm=64, bn=64, bk=32):
    """The kernel for shapes the tiled kernels do not take (any M, N, K and alignment): one element per
    global access, operands staged k-major in LDS with zero fill past the edges."""
    assert bm == 64 and bn == 64 and bk % 16 == 0 and 256 * 8 == bm * bk == bn * bk
    M, N, K = size("M"), size("N"), size("K")
    row, col, kk, sr, sk = (idx(n) for n in ("row", "col", "kk", "sr", "sk"))
    rng = {row: (0, M), col: (0, N), kk: (0, K)}
    flat = lambda lay, i, j: tidy(lay.TileBy([lay.dims()[0], lay.dims()[1]])[i, j], rng)  # noqa: E731
    pitch = bk + 8        # 80-byte rows: eight-k reads of 32 consecutive rows cover every 16-byte bank group evenly
    S = OrderBy(Row(bm, pitch)).TileBy([bm, pitch])
    text = template("gemm_any.hip.j2").render(
        banner=BANNER, BM=bm, BN=bn, BK=bk, PITCH=pitch,
        a_row_layout="OrderBy(Row(M, K))[row, kk]", a_col_layout="OrderBy(Col(M, K))[row, kk]",
        b_row_layout="OrderBy(Row(K, N))[kk, col]", b_col_layout="OrderBy(Col(K, N))[kk, col]",
        c_layout="OrderBy(Row(M, N))[row, col]", s_layout=f"OrderBy(Row({bm}, {pitch}))[sr, sk]",
        a_row=code(flat(OrderBy(Row(M, K)), row, kk)), a_col=code(flat(OrderBy(Col(M, K)), row, kk)),
        b_row=code(flat(OrderBy(Row(K, N)), kk, col)), b_col=code(flat(OrderBy(Col(K, N)), kk, col)),
        c_off=code(flat(OrderBy(Row(M, N)), row, col)),
        s_off=code(tidy(S[sr, sk], {sr: (0, bm), sk: (0, pitch)})))
    return Emitted("gemm_any.hip", text, ["lego_gemm_any_launch"])
