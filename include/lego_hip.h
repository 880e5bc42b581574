/* lego_hip.h -- C ABI of liblego_hip.so, the MI355X (gfx950) kernels generated from LEGO
 * layouts by lego_amd.  Plain pointers and sizes only.
 *
 * Conventions for every entry point
 *   - returns 0 on success, otherwise a hipError_t value (1 = hipErrorInvalidValue for a
 *     null pointer, a misaligned base, or a shape the generated kernels do not cover);
 *   - all tensor pointers are BORROWED DEVICE pointers, row-major and contiguous, aligned to
 *     their element at least (the reference's kernels take any pointer).  16-byte aligned bases
 *     -- what every allocator hands out -- take the fastest kernels; a base at another element (a
 *     sliced view) takes the kernels for rows and shapes of any length, which place their
 *     16-byte accesses where the result has its 16-byte boundaries.  Workspaces and the tuning
 *     entry points (*_wpr, *_split) ask for 16 bytes.  Nothing is allocated, freed or
 *     synchronised: the kernel is enqueued on `stream` (a hipStream_t; NULL = the default
 *     stream) and the call returns;
 *   - re-entrant: safe from several host threads on distinct streams.  Two entry points keep state between
 *     calls, both described where they are declared: lego_hip_lud_f32 (a side stream per caller's stream) and
 *     lego_hip_layernorm_bwd_f16_noalloc (a built-in scratch array per device).
 *
 * The reference has no FFI: its kernels are reached through generated Python host
 * functions.  Each entry point below names the reference host function it stands behind.
 */
#ifndef LEGO_HIP_H
#define LEGO_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

/* ABI version of this header. */
int lego_hip_abi_version(void);

/* out[c][r] = in[r][c] for a rows x cols matrix; out is cols x rows.
 * Replaces the generated transpose programs (reference: benchmarks/mlir/transpose_smem.py:28-80,
 * mlir_generated/transpose/transpose_smem_4096.mlir:24-97), which have no callable entry.
 * Any shape; rows and cols in whole 16-byte vectors (multiples of 8 for 2-byte, of 4 for 4-byte
 * elements) take the 16-byte-per-lane kernels, without edge tests when they are whole tiles;
 * other shapes the same kernels with 16-byte accesses at any element (about two thirds as fast), tiny
 * ones a kernel that moves one element per access.  _f32 moves 4-byte
 * elements, _f16 2-byte elements, whatever their type. */
int lego_hip_transpose_f32(const void* in, void* out, int rows, int cols, void* stream);
int lego_hip_transpose_f16(const void* in, void* out, int rows, int cols, void* stream);

/* y = softmax(x) over the last dimension of an M x N matrix (fp16 or fp32 in/out), fp32
 * arithmetic.  Replaces softmax(x) (reference: triton_generated/softmax/softmax.py:97-160; the
 * reference's own test is a ragged fp32 1823 x 781 matrix, softmax.py:237-241).
 * Any N; rows that are not whole 16-byte vectors are split at their 16-byte boundaries, rows above
 * 16384 elements a whole workgroup of 1024 lanes each, rows above 32768 elements are read twice
 * (the reference keeps a whole row in one block whatever its length, softmax.py:104). */
int lego_hip_softmax_f16(const void* x, void* y, int M, int N, void* stream);
int lego_hip_softmax_f32(const void* x, void* y, int M, int N, void* stream);

/* The same for bfloat16 tensors (the reference's kernel takes the tensor's own type, softmax.py:97-160). */
int lego_hip_softmax_bf16(const void* x, void* y, int M, int N, void* stream);

/* LayerNorm forward over the last dimension of an M x N matrix; x, y, w, b share one element
 * type (fp16, bfloat16 or fp32), w and b have N elements; mean, rstd are fp32 [M] outputs.  Replaces
 * LEGOLayerNorm.forward / lego_layer_norm (reference:
 * triton_generated/layernorm/layernorm.py:279-307, whose limit is 64 KiB of row, :291-294).
 * Any N up to 32768. */
int lego_hip_layernorm_fwd_f16(const void* x, void* y, const void* w, const void* b,
                               float* mean, float* rstd, int M, int N, float eps, void* stream);
int lego_hip_layernorm_fwd_f32(const void* x, void* y, const void* w, const void* b,
                               float* mean, float* rstd, int M, int N, float eps, void* stream);
int lego_hip_layernorm_fwd_bf16(const void* x, void* y, const void* w, const void* b,
                                float* mean, float* rstd, int M, int N, float eps, void* stream);

/* LayerNorm backward: dx (M x N fp16), dw and db (N fp16) from dy, x, w and the forward pass's
 * mean and rstd.  Replaces LEGOLayerNorm.backward (reference:
 * triton_generated/layernorm/layernorm.py:162-268, host side :372-405), whose lock-guarded
 * partial buffers become one fp32 workspace the caller provides (the reference's wrapper
 * allocates its buffers with torch as well): ask for its size first, any 16-byte aligned
 * device buffer of at least that many bytes will do; its contents need no initialisation.
 * Any N up to 32768 (the reference's fp16 limit); rows above 16384 elements are read twice (dx by
 * rows, then dw/db by columns).  Rows of a length that is not a multiple of 8, and tensors at a base that is
 * not 16-byte aligned, are split where the rows of dx have their 16-byte boundaries (the same columns in dy and x
 * when all three are 16-byte aligned buffers of one shape).  The workspace size covers either case. */
int lego_hip_layernorm_bwd_workspace_bytes(int M, int N, unsigned long long* bytes);
int lego_hip_layernorm_bwd_f16(const void* dy, const void* x, const void* w, const float* mean,
                               const float* rstd, void* dx, void* dw, void* db, void* workspace,
                               unsigned long long workspace_bytes, int M, int N, void* stream);

/* lego_hip_layernorm_bwd_f16 without the workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  The fp32 partial rows live in a 32 MiB array inside the library's
 * code object, one copy per device, held until the process ends; every fp16 shape that
 * lego_hip_layernorm_bwd_f16 takes needs at most that much (a shape that needed more would return
 * hipErrorInvalidValue).  The device that owns `stream` must be the current device of the calling
 * thread.  Calls on one device share the array: two calls that overlap in time on one device (on
 * different streams) race on it and must be ordered by the caller.  The call itself allocates and
 * frees nothing and does not synchronise.  The first call on a device looks up the array's device address
 * (hipGetSymbolAddress, which may load the code object that holds the array): make that call outside any
 * stream capture; the calls after it only enqueue kernels and can be captured. */
int lego_hip_layernorm_bwd_f16_noalloc(const void* dy, const void* x, const void* w, const float* mean,
                                       const float* rstd, void* dx, void* dw, void* db, int M, int N, void* stream);

/* The same for fp32 tensors (the reference's kernels take the tensors' own type, layernorm.py:372-405): the
 * kernels of fp16 for rows of up to 16384 elements, two passes above; the workspace has its own size. */
int lego_hip_layernorm_bwd_f32_workspace_bytes(int M, int N, unsigned long long* bytes);
int lego_hip_layernorm_bwd_f32(const void* dy, const void* x, const void* w, const float* mean,
                               const float* rstd, void* dx, void* dw, void* db, void* workspace,
                               unsigned long long workspace_bytes, int M, int N, void* stream);
/* ... and for bfloat16 tensors, with the kernels and the workspace size of fp16. */
int lego_hip_layernorm_bwd_bf16_workspace_bytes(int M, int N, unsigned long long* bytes);
int lego_hip_layernorm_bwd_bf16(const void* dy, const void* x, const void* w, const float* mean,
                                const float* rstd, void* dx, void* dw, void* db, void* workspace,
                                unsigned long long workspace_bytes, int M, int N, void* stream);

/* C = A * B, A is M x K, B is K x N, C is M x N, fp16 with fp32 accumulation.
 * Replaces matmul(a, b) (reference: triton_generated/matmul/matmul_NTA_NTB.py:129-145).
 * Any M, N, K (the reference keeps them symbolic and masks its tiles' edges, matmul_sympy.py:69-70,
 * 196-203).  The MFMA kernels on 256 x 256 (or 128 x 128) tiles, ragged at the edges and with a masked
 * last k-tile where need be, take every shape whose operand rows are whole 16-byte chunks on 16-byte
 * aligned bases: N a multiple of 8, and K (operands as given) or M (A transposed) a multiple of 8 as
 * well.  Any other shape or alignment (bases need only element alignment then) takes a kernel that
 * moves one element per access, about a tenth as fast.  Shapes in whole tiles take a kernel without
 * edge tests. */
int lego_hip_gemm_f16(const void* a, const void* b, void* c, int M, int N, int K, void* stream);
/* The same with the reference's fused epilogue (matmul(a, b, activation="leaky_relu"),
 * matmul_NTA_NTB.py:129-145): activation 0 = none, 1 = leaky_relu on the fp32 accumulator. */
int lego_hip_gemm_f16_act(const void* a, const void* b, void* c, int M, int N, int K, int activation, void* stream);
/* The reference's four operand layouts (matmul_{N,}TA_{N,}TB.py: the operands there are `.T`
 * views, i.e. column-major storage of the same logical matrices): trans_a != 0 means `a` points
 * to a K x M row-major buffer, trans_b != 0 means `b` points to an N x K row-major buffer. */
int lego_hip_gemm_f16_ex(const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                         int activation, void* stream);
/* The same kernel for bfloat16 operands and result (fp32 accumulation).  The reference's matmul
 * takes whatever 16-bit dtype its tensors have and stores fp16 (matmul_sympy.py:129-145, 203);
 * here the result has the operands' type. */
int lego_hip_gemm_bf16_ex(const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                          int activation, void* stream);
/* bfloat16 operands, fp16 result: what the reference's matmul returns for bfloat16 tensors (it stores
 * `accumulator.to(tl.float16)` into a float16 tensor whatever its operands' type, matmul_sympy.py:136, 203). */
int lego_hip_gemm_bf16_f16_ex(const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                              int activation, void* stream);
/* The same products (element: 0 = fp16, 1 = bfloat16, 4 = bfloat16 operands with fp16 result) with room for partial
 * sums.  A product of few tiles -- a skinny operand (16 x 8192 x 8192), a long K (256 x 256 x 65536) -- leaves most
 * CUs idle with one workgroup per tile and cannot pull its operands through the chip; with a workspace the k-tiles
 * of every tile are dealt to several workgroups, which leave fp32 sums there, and a second kernel adds them in a
 * fixed order (deterministic), applies the activation and stores C.  A product with N or K that is not a multiple
 * of 8 (operand rows that are not whole 16-byte chunks) runs on zero-padded copies of A, B and C in the workspace
 * instead of the one-element-per-access kernel, about ten times as fast; operands may then start at any element.
 * lego_hip_gemm_workspace_bytes gives the size the call uses for a shape (0: it gains nothing from a workspace).
 * The workspace is scratch: 16-byte aligned device memory, contents undefined on entry and exit, not to be shared
 * by calls that may overlap.  With a null or short workspace the call is lego_hip_gemm_*_ex.  No counterpart in
 * the reference, whose matmul has one program per tile (matmul_sympy.py:57-65). */
int lego_hip_gemm_workspace_bytes(int M, int N, int K, unsigned long long* bytes);
int lego_hip_gemm_ex_ws(int element, const void* a, const void* b, void* c, int M, int N, int K, int trans_a,
                        int trans_b, int activation, void* workspace, unsigned long long workspace_bytes,
                        void* stream);
/* 8-bit floating-point operands, fp32 accumulation, fp16 result: the reference's fp8 path casts
 * both operands to float8_e5m2 and stores fp16 (matmul_sympy.py:346-364, 203).  format 0 = OCP
 * e4m3 (torch.float8_e4m3fn), 1 = OCP e5m2 (torch.float8_e5m2); a and b hold one byte per
 * element; shapes as for fp16, a 16-byte chunk being 16 elements and a k-tile 128. */
int lego_hip_gemm_fp8_ex(const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                         int activation, int format, void* stream);

/* 3-D stencils on an n x n x n fp32 array (the reference's bricks benchmarks:
 * benchmarks/cuda/bricks_f3d.py:8-22 with bricks/main_tmp.cu:24-104, and bricks_laplasian.py:8-33
 * with bricks-laplace/main_tmp.cu:24-96).  bricks == 0: in and out are row-major; bricks != 0:
 * they are stored as contiguous 8 x 8 x 8 bricks, bricks in row-major order.  Points closer
 * than radius (1..3; the laplacian, which the reference runs up to 4, 1..4) to the boundary are not written.
 * n a multiple of 8, at most 1024.
 *   f3d:        out = in*c[r][r][r] + sum over |di|,|dj|,|dk| <= r of in[+di,+dj,+dk] * c[di+r][dj+r][dk+r],
 *               c an 8 x 8 x 8 array;
 *   laplacian:  out = in*c[0] + sum over a = 1..r of c[a] * (the six neighbours at distance a),
 *               c an array of r+1 floats. */
int lego_hip_stencil_f3d_f32(const float* in, float* out, const float* c, int n, int radius, int bricks, void* stream);
int lego_hip_stencil_laplacian_f32(const float* in, float* out, const float* c, int n, int radius, int bricks,
                                   void* stream);

/* LU decomposition without pivoting of an n x n fp32 row-major matrix, in place: on return the
 * strict lower triangle holds L (unit diagonal implied) and the upper triangle holds U, as
 * Rodinia's lud (the reference's thread-coarsening benchmark: benchmarks/cuda/lud.py:5-12,
 * kernels lud/lud_kernel_temp.cu:14-352, host loop :358-390).  n a multiple of 64, at most 32768.
 * From n = 4928 on, part of the work is enqueued on a second stream, forked from and joined back into
 * `stream` with events inside the call, so the caller sees ordinary stream order (captured into a graph,
 * the fork and join become graph edges).  The library makes that stream and its two events on the first
 * such call for a given (device, `stream`) pair -- the device of `stream` must be current -- and keeps
 * them until the process ends: callers on distinct streams share nothing.  After 32 such pairs, and for a
 * `stream` that is under capture the first time it is seen (nothing is created during a capture), the
 * call stays on `stream` alone (same results, less overlap).  Concurrent calls on the SAME `stream` from
 * several threads are not supported, as for any stream-ordered work. */
int lego_hip_lud_f32(float* m, int n, void* stream);

/* The launches that lego_hip_lud_f32 enqueues for an n x n matrix, in order, without touching a device: six
 * ints per launch, {kind, stream, a, b, c, d}, stream 0 = the caller's, 1 = the library's second one.
 *   kind 0 panels of step a (b workgroups);  1 strip: block row and column a+1 against step a (b = blocks left in
 *   a block row);  2 the two block rows and columns at the top and left of the square of side c from block b on,
 *   against steps a, a+1;  3 trailing update of the square of side c from block b on against d/16 steps from a on,
 *   d%16 blocks per workgroup;  4 fork (stream 1 waits for stream 0);  5 join (stream 0 waits for stream 1);
 *   6 factors of the a diagonal blocks written.
 * At most `capacity` records are written; *count receives how many there are.  No counterpart in the
 * reference (its host loop, lud_kernel_temp.cu:358-390, is three launches per step on one stream): it is
 * there so that the order and the overlap of the launches can be checked on the host. */
int lego_hip_lud_f32_plan(int n, int* records, int capacity, int* count);

/* Needleman-Wunsch score matrix (Rodinia's needle, the reference's anti-diagonal layout
 * benchmark: benchmarks/cuda/nw_sympy.py:9-11, kernels needle_kernel_temp.cu:70-258, host
 * needle.cu:165-260).  reference and matrix are (n+1) x (n+1) int32, row-major; row 0 and
 * column 0 of matrix hold the borders (-i*penalty in Rodinia); on return
 * matrix[i][j] = max(matrix[i-1][j-1] + reference[i][j], matrix[i][j-1] - penalty,
 * matrix[i-1][j] - penalty) for i, j >= 1.  n a multiple of 64, at most 32768. */
int lego_hip_nw_i32(const int* reference, int* matrix, int n, int penalty, void* stream);

/* groups independent GEMMs in one launch.  a, b, c are HOST arrays of `groups` device
 * pointers; sizes3 is a HOST array of groups*3 ints (M, N, K per problem).  Any number of
 * groups: one launch carries up to 64 problems (their pointers and sizes travel as kernel arguments), a
 * call with more is enqueued as runs of 64 in order of decreasing K, one launch after the other on
 * `stream`.  One launch per run when every N and K is a multiple of 8 and every base 16-byte aligned (any M;
 * ragged tiles and last k-tiles are masked); otherwise one launch per problem, as lego_hip_gemm_f16
 * would take it.  Replaces
 * lego_group_gemm_fn(group_A, group_B) (reference:
 * triton_generated/grouped_gemm/grouped_gemm.py:120-162), whose device-side tables are
 * passed here by value as kernel arguments, so no table is allocated or copied. */
int lego_hip_grouped_gemm_f16(const void* const* a, const void* const* b, void* const* c,
                              const int* sizes3, int groups, void* stream);

/* What lego_hip_grouped_gemm_f16 launches for these sizes, without touching a device: plan3[0] = tile
 * size (256: 256 x 256 tiles, or 128: 128 x 128 tiles), plan3[1] = number of 256 x 256 tiles of all
 * problems, plan3[2] = how many of them, the last ones of the launch order, are computed as two
 * 128 x 256 halves by two workgroups.  At most 64 groups (one launch).  No counterpart in the reference (its kernel walks whole tiles
 * only, grouped_gemm.py:61-116); it is there so that the launch can be checked on the host. */
int lego_hip_grouped_gemm_f16_plan(const int* sizes3, int groups, int* plan3);
/* Tuning entry point: lego_hip_grouped_gemm_f16 with the launch chosen by the caller: split_tiles >= 0
 * = 256 x 256 tiles, the last split_tiles of them as halves; split_tiles < 0 = 128 x 128 tiles. */
int lego_hip_grouped_gemm_f16_split(const void* const* a, const void* const* b, void* const* c,
                                    const int* sizes3, int groups, int split_tiles, void* stream);

/* Tuning entry points: the transposes with the tiling chosen by the caller, by its place in the library's list of
 * tilings for the element type (lego_amd/build.py, TRANSPOSE; 0 = the first).  Invalid value if the list has no such
 * entry or the shape is not one that tiling takes (whole windows of macro tiles for the first ones); bases 16-byte
 * aligned.  Used by the benchmark to compare tilings on one shape.  No counterpart in the reference. */
int lego_hip_transpose_f32_tiling(const void* in, void* out, int rows, int cols, int tiling, void* stream);
int lego_hip_transpose_f16_tiling(const void* in, void* out, int rows, int cols, int tiling, void* stream);

/* Tuning entry points: as above, with the launch shape chosen by the caller
 * (waves_per_row in {1, 2, 4, 8, 16}; N a multiple of 8 and at most 8192 * waves_per_row, 16384 for 4 and 8).  Used by the benchmark to compare variants. */
int lego_hip_softmax_f16_wpr(const void* x, void* y, int M, int N, int waves_per_row, void* stream);
int lego_hip_layernorm_fwd_f16_wpr(const void* x, void* y, const void* w, const void* b,
                                   float* mean, float* rstd, int M, int N, float eps,
                                   int waves_per_row, void* stream);

/* What lego_hip_gemm_f16_ex and lego_hip_gemm_bf16*_ex launch for a product whose operands lie in whole 16-byte chunks,
 * without touching a device: plan2[0] = side of the workgroup's tile (256 or 128), plan2[1] = side of the MFMA's
 * accumulator block (16: v_mfma_f32_16x16x32, 32: v_mfma_f32_32x32x16).  No counterpart in the reference (its
 * autotuner picks among tile configurations at run time, matmul_sympy.py:98-165); it is there so that the choice can be
 * checked on the host. */
int lego_hip_gemm_plan(int M, int N, int K, int* plan2);

/* The team that lego_hip_softmax_f16 and lego_hip_layernorm_fwd_f16 give a row of a matrix of M rows of N fp16
 * elements in whole 16-byte vectors on 16-byte aligned bases (N a multiple of 8, at most 32768): waves per row, the
 * argument that the _wpr entry points above take.  Host only; no counterpart in the reference (its softmax sizes one
 * program from BLOCK_SIZE with a fixed num_warps = 8, softmax.py:97-122). */
int lego_hip_rows_f16_plan(int M, int N, int* waves_per_row);

/* Tuning entry point: C = A * B (fp16, row-major, N and K multiples of 8, 16-byte aligned bases) on 256 x 256 tiles
 * with the kernel chosen by the caller: variant 0 = what lego_hip_gemm_f16 launches for large products (four waves of
 * 128 x 128, one per SIMD with 256 accumulator registers, v_mfma_f32_16x16x32_f16), 1 = the same workgroup with
 * v_mfma_f32_32x32x16_f16 (what it launches for 129 to 175 tiles, one round of workgroups that leaves a third of the
 * CUs idle), 2 = eight waves of 128 x 64, two per SIMD with 128 accumulator registers each
 * (v_mfma_f32_32x32x16_f16), 3 = the measurement build of variant 0 (below).  Used by the benchmark to compare
 * them.  No counterpart in the reference. */
int lego_hip_gemm_f16_variant(const void* a, const void* b, void* c, int M, int N, int K, int variant, void* stream);

/* Measurement aid (no counterpart in the reference): where the time of a tile goes.  A second build of the fp16
 * 256 x 256-tile kernels, plain and grouped, same tiles and instruction schedules, in which lane 0 of every
 * workgroup with an id below 8192 stores the 100 MHz real-time counter at seven points of its tile and, once,
 * where it ran.  lego_hip_gemm_f16_variant(..., 3, ...) launches the plain kernel,
 * lego_hip_grouped_gemm_f16_stamps the grouped one with the launch that lego_hip_grouped_gemm_f16 would choose
 * (at most 64 problems in whole tiles; a problem set that the entry point would give to the 128 x 128 tiles is refused).
 * lego_hip_gemm_stamps_read copies the rows of the first `workgroups` workgroup ids of the last such launch to the
 * host (eight 64-bit words each; it synchronises with the device): words 0..6 = entry, first k-tile in LDS, first
 * fragments read, main loop and the k-tile before the last done, the last k-tile's slots issued, the last stores
 * issued, the stores gone; word 7 = the hardware id of the wave (bits 0-15: HW_ID with SIMD, CU, shader array and
 * engine) and the XCD (bits 16-19).  bench.py --only timeline prints the per-phase table. */
int lego_hip_grouped_gemm_f16_stamps(const void* const* a, const void* const* b, void* const* c,
                                     const int* sizes3, int groups, void* stream);
int lego_hip_gemm_stamps_read(unsigned long long* host, int workgroups);

/* Measurement aid: out[0..bytes) = in[0..bytes), 16 bytes per lane per access, bytes % 16 == 0.
 * No counterpart in the reference.  bench.py uses it as the same-run copy ceiling and the
 * profiles use it to calibrate the FETCH_SIZE / WRITE_SIZE counters at this access width. */
int lego_hip_copy16(const void* in, void* out, unsigned long long bytes, void* stream);
/* Streaming copy (no counterpart in the reference): non-temporal accesses, one contiguous 16 KiB
 * chunk per workgroup -- the access pattern of the row kernels without their arithmetic, i.e.
 * the bandwidth a kernel that reads and writes every byte once can reach on this part.
 * bytes a multiple of 16384. */
int lego_hip_copy16_stream(const void* in, void* out, unsigned long long bytes, void* stream);

/* Measurement aid (no counterpart in the reference): what the memory delivers to a stream in one direction, in
 * the access shape of lego_hip_copy16_stream -- non-temporal 16-byte accesses, vectors_per_lane (1 or 4) of them
 * per lane, one contiguous chunk of 4 KiB * vectors_per_lane per workgroup of 256 lanes.
 *   mode 0: read in[0..bytes) and store next to nothing (a lane's words are folded and compared with a constant;
 *           a lane that matches, one in 2^32 for random data, stores one vector into the first 4 KiB of out);
 *           mode 1: write out[0..bytes), in is not read;
 *   mode 2: out[0..bytes) = in[0..bytes).
 * bytes a multiple of the chunk.  bench.py times modes 0 and 1 on rotating 512 MiB buffers and derives from them
 * the rate that a kernel which reads and writes every byte once cannot pass on this part. */
int lego_hip_hbm_probe(const void* in, void* out, unsigned long long bytes, int mode, int vectors_per_lane, void* stream);

/* Measurement aid (no counterpart in the reference): what the matrix cores sustain when a kernel does nothing but
 * issue MFMAs.  `workgroups` workgroups of four waves (one per SIMD, 256 accumulator registers each, the occupancy
 * of the GEMM kernels); a wave loads sixteen 16-byte operand fragments per lane once (operands: workgroups * 64 KiB
 * of 16-bit values, the caller's choice of distribution: the power a matrix core draws depends on its data) and
 * runs `iters` rounds of MFMAs over a 128 x 128 block of accumulators: one MFMA per accumulator block and round,
 * so a round is a k-step of the instruction's depth.
 *   shape 0: v_mfma_f32_32x32x16_f16 (16 per round and wave: 2097152 flop per round and workgroup)
 *   shape 1: v_mfma_f32_16x16x32_f16 (64 per round and wave: 4194304 flop per round and workgroup)
 *   shape 2: v_mfma_f32_32x32x16_bf16 (the same bits read as bfloat16; flop as shape 0)
 *   shape 3 / 4: the instructions of shapes 1 / 0 with two waves per SIMD (workgroups of eight waves with 128
 *   accumulator registers each, a 128 x 64 block per wave: 4194304 / 2097152 flop per round and workgroup).
 *   shape 5 / 6: v_mfma_f32_32x32x64_f8f6f4 with the operands' bytes read as OCP e5m2 / e4m3 (16 per round and
 *   wave over 4 x 4 blocks: 8388608 flop per round and workgroup; the same workgroups * 64 KiB of operands).
 *   shape 7: v_mfma_f32_16x16x128_f8f6f4 on the operands of shape 5 (e5m2; 64 per round and wave over 8 x 8 blocks:
 *   16777216 flop per round and workgroup).
 * sink: workgroups * 512 floats (a sum per lane, so that the work is not optimised away).  bench.py runs it with
 * operands of the GEMM benchmark's distribution and reports the rate as what the socket's power limit leaves to
 * an fp16 GEMM whose data movement costs nothing. */
int lego_hip_mfma_probe(const void* operands, float* sink, int shape, int iters, int workgroups, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LEGO_HIP_H */
