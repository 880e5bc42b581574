"""The reference's two transpose programs, written against the HIP kernel builder.

``transpose_naive`` and ``transpose_smem`` state the same layouts and the same
per-thread work as benchmarks/mlir/transpose_naive.py:26-58 and
benchmarks/mlir/transpose_smem.py:28-80 (32x32 tiles, 256 threads, four elements per
thread, a one-dimensional grid decoded row-major for reads and column-major for
writes).  They exist for parity with the reference's generated programs and as the
scalar baseline the vectorised transpose of ``lego_amd.kernels.transpose`` is measured
against; the benchmark repetitions and host allocation that the reference puts inside
the generated program are left to the caller.
"""
from ..lego_hip import HipTensor, printer
from ..lego import Col, OrderBy, Row

TILE_DIM = 32
BLOCK_ROWS_X = 8
BLOCK_ROWS_Y = 32


def _ids(n):
    """Tile and thread coordinates for the read side (row-major) and the write side
    (column-major) of the one-dimensional launch."""
    nb = n // TILE_DIM
    bX = printer.get_block_linear_index()
    tX = printer.get_thread_linear_index()
    read_tile = OrderBy(Row(nb, nb)).TileBy([nb, nb]).inv(bX)
    write_tile = OrderBy(Col(nb, nb)).TileBy([nb, nb]).inv(bX)
    read_thread = OrderBy(Row(BLOCK_ROWS_X, BLOCK_ROWS_Y)).TileBy([BLOCK_ROWS_X, BLOCK_ROWS_Y]).inv(tX)
    write_thread = OrderBy(Col(BLOCK_ROWS_Y, BLOCK_ROWS_X)).TileBy([BLOCK_ROWS_Y, BLOCK_ROWS_X]).inv(tX)
    return read_tile, write_tile, read_thread, write_thread


def _tiled(n, inner):
    nb = n // TILE_DIM
    return OrderBy(Row(n, n)).TileBy([nb, nb], [TILE_DIM // inner[0], TILE_DIM // inner[1]], inner)


def transpose_naive(n, dtype="f32"):
    """``B[c][r] = A[r][c]`` straight through global memory."""
    grid, block = (n // TILE_DIM * n // TILE_DIM, 1, 1), (BLOCK_ROWS_X * BLOCK_ROWS_Y, 1, 1)

    @printer.generate_hip(name=f"lego_dsl_transpose_naive_{dtype}_{n}")
    def module():
        TA = HipTensor(_tiled(n, [BLOCK_ROWS_X, BLOCK_ROWS_Y]), dtype)
        TB = HipTensor(_tiled(n, [BLOCK_ROWS_Y, BLOCK_ROWS_X]), dtype)

        @printer.generate_gpu_kernel([TA], [TB], grid, block)
        def kernel(_):
            (rby, rbx), (wby, wbx), (rty, rtx), (wty, wtx) = _ids(n)
            steps = [TILE_DIM // BLOCK_ROWS_X, TILE_DIM // BLOCK_ROWS_Y]

            @printer.generate_loop(OrderBy(Row(*steps)).TileBy(steps))
            def body(pargs, _):
                j, i = pargs
                TB[wby, wbx, i, j, wty, wtx] = TA[rby, rbx, j, i, rty, rtx]
    return module


def transpose_smem(n, dtype="f32"):
    """The same through a 32x32 staging tile whose layout is re-stated between the
    write phase and the read phase."""
    grid, block = (n // TILE_DIM * n // TILE_DIM, 1, 1), (BLOCK_ROWS_X * BLOCK_ROWS_Y, 1, 1)

    def staging(inner):
        return OrderBy(Row(TILE_DIM, TILE_DIM)).TileBy(
            [TILE_DIM // inner[0], TILE_DIM // inner[1]], inner)

    @printer.generate_hip(name=f"lego_dsl_transpose_smem_{dtype}_{n}")
    def module():
        TA = HipTensor(_tiled(n, [BLOCK_ROWS_X, BLOCK_ROWS_Y]), dtype)
        TB = HipTensor(_tiled(n, [BLOCK_ROWS_X, BLOCK_ROWS_Y]), dtype)
        TS = HipTensor(OrderBy(Row(TILE_DIM, TILE_DIM)).TileBy([TILE_DIM, TILE_DIM]), dtype)

        @printer.generate_gpu_kernel([TA], [TB], grid, block, workgroup_memory=[TS])
        def kernel(_):
            (rby, rbx), (wby, wbx), (rty, rtx), (wty, wtx) = _ids(n)

            TS.layout = staging([BLOCK_ROWS_X, BLOCK_ROWS_Y])
            fill = [TILE_DIM // BLOCK_ROWS_X, TILE_DIM // BLOCK_ROWS_Y]

            @printer.generate_loop(OrderBy(Row(*fill)).TileBy(fill))
            def stage(pargs, _):
                j, i = pargs
                TS[j, i, rty, rtx] = TA[rby, rbx, j, i, rty, rtx]

            printer.insert_barrier()

            TS.layout = staging([BLOCK_ROWS_Y, BLOCK_ROWS_X])
            drain = [TILE_DIM // BLOCK_ROWS_Y, TILE_DIM // BLOCK_ROWS_X]

            @printer.generate_loop(OrderBy(Row(*drain)).TileBy(drain))
            def unstage(pargs, _):
                j, i = pargs
                TB[wby, wbx, i, j, rty, rtx] = TS[j, i, wty, wtx]
    return module


def row_sums(rows, cols, dtype="f32"):
    """``out[r] = sum_c A[r][c]``: a loop that carries its running sum, the builder's counterpart of the
    reference's ``affine.for ... iter_args`` (lego/lego_mlir.py:85-108).  One lane per row, 64 lanes per
    workgroup; no reference program uses a carried value, this one exists to exercise that path."""
    assert rows % 64 == 0
    grid, block = (rows // 64, 1, 1), (64, 1, 1)

    @printer.generate_hip(name=f"lego_dsl_row_sums_{dtype}_{rows}x{cols}")
    def module():
        TA = HipTensor(OrderBy(Row(rows, cols)).TileBy([rows // 64, 1], [64, cols]), dtype)
        TS = HipTensor(OrderBy(Row(rows)).TileBy([rows // 64], [64]), dtype)

        @printer.generate_gpu_kernel([TA], [TS], grid, block)
        def kernel(_):
            bX = printer.get_block_linear_index()
            tX = printer.get_thread_linear_index()

            @printer.generate_loop(OrderBy(Row(cols)).TileBy([cols]), iter_args=[0.0])
            def total(pargs, _, carried):
                (c,) = pargs
                return carried[0] + TA[bX, 0, tX, c]
            (acc,) = total()
            TS[bX, tX] = acc
    return module
