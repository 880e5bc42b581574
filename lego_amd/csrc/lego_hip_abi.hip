// C-ABI entry points of liblego_hip.so (declared in include/lego_hip.h).
//
// This file is written by hand; the kernels and their launchers are generated from LEGO
// layouts (python -m lego_amd.build) into csrc/generated/ and declared in
// generated/launchers.h.  An entry point validates what the generated code assumes --
// non-null, 16-byte aligned pointers and shapes that divide the tiles -- and enqueues one
// kernel on the caller's stream.  It allocates nothing and never synchronises.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string.h>

#include <algorithm>
#include <mutex>
#include <vector>

#include "lego_hip.h"
#include "generated/launchers.h"

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool usable(const void* p) { return p != nullptr && aligned16(p); }
// a tensor base that only has its elements' alignment (a sliced view): the kernels for rows and shapes of any
// length take those, with 16-byte accesses wherever their result has its 16-byte boundaries
inline bool element_aligned(const void* p, unsigned bytes) { return p != nullptr && (reinterpret_cast<uintptr_t>(p) & (bytes - 1u)) == 0; }
inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }
inline int ok_or(hipError_t e) { return static_cast<int>(e); }
constexpr int kInvalid = static_cast<int>(hipErrorInvalidValue);

// plain grid-stride copy, one 16-byte vector per lane per step
__global__ void __launch_bounds__(256) lego_copy16_kernel(const uint4* __restrict__ in, uint4* __restrict__ out, size_t n)
{
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = in[i];
}

// streaming copy: a workgroup owns one contiguous 16 KiB chunk, four non-temporal 16-byte loads
// per lane in flight, then four non-temporal stores
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) lego_copy16_stream_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out)
{
  const size_t base = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
  u32x4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(in + base + u * 256);
#pragma unroll
  for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(v[u], out + base + u * 256);
}

// What the memory delivers to one-directional streams, in the access shape of lego_copy16_stream_kernel (V
// non-temporal 16-byte vectors per lane, a contiguous V*4 KiB chunk per workgroup): a read-only stream whose
// values are folded into one word and compared with a constant (the loads must depend on the data, or the
// compiler drops them; a lane whose words happen to fold to the constant stores one vector into the first 4 KiB
// of `sink`), and a write-only stream of a lane-dependent pattern.
template <int V>
__global__ void __launch_bounds__(256) lego_probe_read_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ sink)
{
  const size_t base = static_cast<size_t>(blockIdx.x) * (256 * V) + threadIdx.x;
  u32x4 v[V];
#pragma unroll
  for (int u = 0; u < V; ++u) v[u] = __builtin_nontemporal_load(in + base + u * 256);
  unsigned acc = 0;
#pragma unroll
  for (int u = 0; u < V; ++u) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  if (acc == 0x9e3779b9u) sink[threadIdx.x] = v[0];
}
template <int V>
__global__ void __launch_bounds__(256) lego_probe_write_kernel(u32x4* __restrict__ out)
{
  const size_t base = static_cast<size_t>(blockIdx.x) * (256 * V) + threadIdx.x;
  const u32x4 v = {threadIdx.x, blockIdx.x, 3u, 4u};
#pragma unroll
  for (int u = 0; u < V; ++u) __builtin_nontemporal_store(v, out + base + u * 256);
}
template <int V>
__global__ void __launch_bounds__(256) lego_probe_copy_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out)
{
  const size_t base = static_cast<size_t>(blockIdx.x) * (256 * V) + threadIdx.x;
  u32x4 v[V];
#pragma unroll
  for (int u = 0; u < V; ++u) v[u] = __builtin_nontemporal_load(in + base + u * 256);
#pragma unroll
  for (int u = 0; u < V; ++u) __builtin_nontemporal_store(v[u], out + base + u * 256);
}

// What the matrix cores sustain when nothing else happens: every wave of a workgroup of four (one per SIMD, 256
// accumulator registers, as in the GEMM kernels) loads sixteen operand fragments once and then issues nothing but
// MFMAs on them, a 128 x 128 block of accumulators per wave.  With random operands this is the rate the socket's
// power limit leaves to a GEMM whose loads, LDS traffic and address arithmetic cost nothing.
typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef __bf16 probe_bhalf8 __attribute__((ext_vector_type(8)));
typedef float probe_float16 __attribute__((ext_vector_type(16)));
typedef float probe_float4 __attribute__((ext_vector_type(4)));
// The same with two waves per SIMD (workgroups of eight waves, 128 accumulator registers each, a 128 x 64 block):
// whether a second wave to issue from changes what the pipe sustains.
template <int SHAPE>      // 3: v_mfma_f32_16x16x32_f16 (8 x 4 blocks)  4: v_mfma_f32_32x32x16_f16 (4 x 2 blocks)
__global__ void __launch_bounds__(512) lego_mfma_probe2_kernel(const probe_half8* __restrict__ operands, float* __restrict__ sink, unsigned iters)
{
  const probe_half8* mine = operands + (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x % 256) * 16;
  probe_half8 fa[8], fb[4];
#pragma unroll
  for (int f = 0; f < 8; ++f) fa[f] = mine[f];
#pragma unroll
  for (int f = 0; f < 4; ++f) fb[f] = mine[8 + f];
  float total = 0.0f;
  if (SHAPE == 3) {
    probe_float4 acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = probe_float4{0.0f, 0.0f, 0.0f, 0.0f};
    for (unsigned it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  } else {
    probe_float16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    for (unsigned it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) total += acc[i][j][r];
  }
  sink[static_cast<size_t>(blockIdx.x) * 512 + threadIdx.x] = total;
}

template <int SHAPE>      // 0: v_mfma_f32_32x32x16_f16 (4 x 4 blocks)  1: v_mfma_f32_16x16x32_f16 (8 x 8 blocks)  2: v_mfma_f32_32x32x16_bf16
__global__ void __launch_bounds__(256) lego_mfma_probe_kernel(const probe_half8* __restrict__ operands, float* __restrict__ sink, unsigned iters)
{
  constexpr int T = SHAPE == 1 ? 8 : 4;
  const probe_half8* mine = operands + (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 16;
  probe_half8 fa[8], fb[8];
#pragma unroll
  for (int f = 0; f < 8; ++f) { fa[f] = mine[f]; fb[f] = mine[8 + f]; }
  float total = 0.0f;
  if (SHAPE == 1) {
    probe_float4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = probe_float4{0.0f, 0.0f, 0.0f, 0.0f};
    for (unsigned it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  } else {
    probe_float16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    for (unsigned it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < T; ++i)
#pragma unroll
        for (int j = 0; j < T; ++j) {
          if (SHAPE == 0) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
          else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(probe_bhalf8, fb[j]), __builtin_bit_cast(probe_bhalf8, fa[i]), acc[i][j], 0, 0, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) total += acc[i][j][r];
  }
  sink[static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x] = total;
}

// 8-bit operands: v_mfma_f32_32x32x64_f8f6f4 on 4 x 4 blocks, the operands' bits read as OCP e5m2 (shape 5) or e4m3 (6)
typedef int probe_int8 __attribute__((ext_vector_type(8)));
template <int FORMAT>     // 0: e4m3  1: e5m2 (the instruction's format codes)
__global__ void __launch_bounds__(256) lego_mfma_probe_8bit_kernel(const probe_int8* __restrict__ operands, float* __restrict__ sink, unsigned iters)
{
  const probe_int8* mine = operands + (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
  probe_int8 fa[4], fb[4];
#pragma unroll
  for (int f = 0; f < 4; ++f) { fa[f] = mine[f]; fb[f] = mine[4 + f]; }
  probe_float16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  for (unsigned it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], acc[i][j], FORMAT, FORMAT, 0, 0, 0, 0);
  }
  float total = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) total += acc[i][j][r];
  sink[static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x] = total;
}

// The same operands through v_mfma_f32_16x16x128_f8f6f4 on 8 x 8 blocks (shape 7): the fragments of the second four
// block rows and columns are those of the first four with their halves swapped, in registers of their own
__global__ void __launch_bounds__(256) lego_mfma_probe_8bit_16x16_kernel(const probe_int8* __restrict__ operands, float* __restrict__ sink, unsigned iters)
{
  const probe_int8* mine = operands + (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
  probe_int8 fa[8], fb[8];
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    fa[f] = mine[f];
    fb[f] = mine[4 + f];
    fa[4 + f] = __builtin_shufflevector(fa[f], fa[f], 4, 5, 6, 7, 0, 1, 2, 3);
    fb[4 + f] = __builtin_shufflevector(fb[f], fb[f], 4, 5, 6, 7, 0, 1, 2, 3);
  }
  probe_float4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = probe_float4{0.0f, 0.0f, 0.0f, 0.0f};
  for (unsigned it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[j], fa[i], acc[i][j], 1, 1, 0, 0, 0, 0);
  }
  float total = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) total += acc[i][j][r];
  sink[static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x] = total;
}

typedef unsigned u32x4w __attribute__((ext_vector_type(4)));
typedef unsigned u32x4w_any __attribute__((ext_vector_type(4), aligned(2)));     // the same 16 bytes at any 2-byte element

// Zero-padded copy of a rows x cols matrix of 2-byte elements (rows at any element alignment) into a
// rows_to x cols_to one with cols_to a multiple of 8 on a 16-byte aligned base: one lane per 16-byte chunk of
// the destination, a source chunk that lies inside its row as a whole is one 16-byte access.
__global__ void __launch_bounds__(256) lego_pad2d_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                         unsigned rows, unsigned cols, unsigned rows_to, unsigned cols_to)
{
  const unsigned per_row = cols_to / 8;
  const size_t chunk = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t r = chunk / per_row;
  const unsigned c = static_cast<unsigned>(chunk % per_row) * 8;
  if (r >= rows_to) return;
  u32x4w v = {0u, 0u, 0u, 0u};
  if (r < rows) {
    const uint16_t* p = src + r * cols + c;
    if (c + 8 <= cols) {
      v = *reinterpret_cast<const u32x4w_any*>(p);
    } else {
#pragma unroll
      for (unsigned e = 0; e < 8; ++e)
        if (c + e < cols) v[e / 2] |= static_cast<uint32_t>(p[e]) << (16 * (e % 2));
    }
  }
  *reinterpret_cast<u32x4w*>(dst + r * cols_to + c) = v;
}

// The way back for the result: rows x cols elements out of a matrix whose rows are cols_from elements apart.
__global__ void __launch_bounds__(256) lego_unpad2d_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                           unsigned rows, unsigned cols, unsigned cols_from)
{
  const unsigned per_row = (cols + 7) / 8;
  const size_t chunk = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t r = chunk / per_row;
  const unsigned c = static_cast<unsigned>(chunk % per_row) * 8;
  if (r >= rows) return;
  const u32x4w v = *reinterpret_cast<const u32x4w*>(src + r * cols_from + c);
  uint16_t* q = dst + r * cols + c;
  if (c + 8 <= cols) {
    *reinterpret_cast<u32x4w_any*>(q) = v;
  } else {
#pragma unroll
    for (unsigned e = 0; e < 8; ++e)
      if (c + e < cols) q[e] = static_cast<uint16_t>(v[e / 2] >> (16 * (e % 2)));
  }
}

hipError_t pad2d(const void* src, void* dst, int rows, int cols, int rows_to, int cols_to, hipStream_t stream)
{
  const size_t chunks = static_cast<size_t>(rows_to) * (cols_to / 8);
  hipLaunchKernelGGL(lego_pad2d_kernel, dim3(static_cast<unsigned>((chunks + 255) / 256)), dim3(256), 0, stream,
                     static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), static_cast<unsigned>(rows),
                     static_cast<unsigned>(cols), static_cast<unsigned>(rows_to), static_cast<unsigned>(cols_to));
  return hipGetLastError();
}

hipError_t unpad2d(const void* src, void* dst, int rows, int cols, int cols_from, hipStream_t stream)
{
  const size_t chunks = static_cast<size_t>(rows) * ((cols + 7) / 8);
  hipLaunchKernelGGL(lego_unpad2d_kernel, dim3(static_cast<unsigned>((chunks + 255) / 256)), dim3(256), 0, stream,
                     static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), static_cast<unsigned>(rows),
                     static_cast<unsigned>(cols), static_cast<unsigned>(cols_from));
  return hipGetLastError();
}

// Scratch of lego_hip_layernorm_bwd_f16_noalloc: the fp32 dw/db partial rows that the other
// LayerNorm backward entry points take from the caller.  One copy per device, held until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress; kernels and launchers
// receive the device address kept in scratch_ptr[device].
constexpr unsigned long long kScratchBytes = 32ull << 20;
static __device__ __align__(256) float scratch[kScratchBytes / sizeof(float)];
constexpr int kMaxDevices = 64;
float* scratch_ptr[kMaxDevices];
std::mutex scratch_mutex;

// Device address of the current device's scratch array (looked up on the first call per device).
hipError_t scratch_address(float** out)
{
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> hold(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return err;
    if (p == nullptr) return hipErrorInvalidSymbol;
    scratch_ptr[dev] = static_cast<float*>(p);
  }
  *out = scratch_ptr[dev];
  return hipSuccess;
}

}  // namespace

extern "C" {

int lego_hip_abi_version(void) { return 1; }

int lego_hip_transpose_f32(const void* in, void* out, int rows, int cols, void* stream)
{
  if (!element_aligned(in, 4) || !element_aligned(out, 4) || in == out) return kInvalid;
  if (rows <= 0 || cols <= 0) return kInvalid;
  if (!aligned16(in) || !aligned16(out))      // a base at any element: the kernels whose vectors sit at any element
    return ok_or(lego_transpose_f32_dispatch_any_base(in, out, rows, cols, as_stream(stream)));
  return ok_or(lego_transpose_f32_dispatch(in, out, rows, cols, as_stream(stream)));
}

int lego_hip_transpose_f16(const void* in, void* out, int rows, int cols, void* stream)
{
  if (!element_aligned(in, 2) || !element_aligned(out, 2) || in == out) return kInvalid;
  if (rows <= 0 || cols <= 0) return kInvalid;
  if (!aligned16(in) || !aligned16(out))
    return ok_or(lego_transpose_f16_dispatch_any_base(in, out, rows, cols, as_stream(stream)));
  return ok_or(lego_transpose_f16_dispatch(in, out, rows, cols, as_stream(stream)));
}

int lego_hip_transpose_f32_tiling(const void* in, void* out, int rows, int cols, int tiling, void* stream)
{
  if (!aligned16(in) || !aligned16(out) || in == out || rows <= 0 || cols <= 0) return kInvalid;
  return ok_or(lego_transpose_f32_tiling(tiling, in, out, rows, cols, as_stream(stream)));
}

int lego_hip_transpose_f16_tiling(const void* in, void* out, int rows, int cols, int tiling, void* stream)
{
  if (!aligned16(in) || !aligned16(out) || in == out || rows <= 0 || cols <= 0) return kInvalid;
  return ok_or(lego_transpose_f16_tiling(tiling, in, out, rows, cols, as_stream(stream)));
}

int lego_hip_softmax_f16_wpr(const void* x, void* y, int M, int N, int waves_per_row, void* stream)
{
  if (!usable(x) || !usable(y)) return kInvalid;
  if (M <= 0 || N <= 0 || N % 8 || N > LEGO_ROWWISE_MAX_N) return kInvalid;
  switch (waves_per_row) {
    case 1:   // rows of at most 16 or 32 vectors: several rows per wave
      return ok_or((N <= 128 ? lego_softmax_f16_l16_launch : N <= 256 ? lego_softmax_f16_l32_launch : lego_softmax_f16_w1_launch)(
          x, y, M, N, as_stream(stream)));
    case 2: return ok_or(lego_softmax_f16_w2_launch(x, y, M, N, as_stream(stream)));
    case 4: return ok_or(lego_softmax_f16_w4_launch(x, y, M, N, as_stream(stream)));
    case 8: return ok_or(lego_softmax_f16_w8_launch(x, y, M, N, as_stream(stream)));
    case 16: return ok_or(lego_softmax_f16_w16_launch(x, y, M, N, as_stream(stream)));
    default: return kInvalid;
  }
}

int lego_hip_softmax_f16(const void* x, void* y, int M, int N, void* stream)
{
  if (!element_aligned(x, 2) || !element_aligned(y, 2) || M <= 0 || N <= 0) return kInvalid;
  if (N > LEGO_ROWWISE_MAX_N) return ok_or(lego_softmax_long_f16_launch(x, y, M, N, as_stream(stream)));   // two passes
  const bool long_row = N > LEGO_ROWWISE_MAX_N_SMALL_TEAMS;
  if (N % 8 || !aligned16(x) || !aligned16(y))   // rows of any length, or at any element
    return ok_or((N <= 128 ? lego_softmax_f16s_l16_launch : N <= 256 ? lego_softmax_f16s_l32_launch
                  : lego_rowwise_f16_wpr(M, N) == 8 ? lego_softmax_f16s_w8_launch
                  : long_row ? lego_softmax_f16s_w16_launch : lego_rowwise_default_wpr(N) == 1 ? lego_softmax_f16s_w1_launch
                                                                                           : lego_softmax_f16s_w4_launch)(
        x, y, M, N, as_stream(stream)));
  return lego_hip_softmax_f16_wpr(x, y, M, N, lego_rowwise_f16_wpr(M, N), stream);
}

int lego_hip_softmax_f32(const void* x, void* y, int M, int N, void* stream)
{
  if (!element_aligned(x, 4) || !element_aligned(y, 4) || M <= 0 || N <= 0) return kInvalid;
  if (N > LEGO_ROWWISE_MAX_N) return ok_or(lego_softmax_long_f32_launch(x, y, M, N, as_stream(stream)));   // two passes
  const bool long_row = N > LEGO_ROWWISE_MAX_N_SMALL_TEAMS;
  if (N % 4 || !aligned16(x) || !aligned16(y))   // rows of any length, or at any element
    return ok_or((N <= 64 ? lego_softmax_f32s_l16_launch : N <= 128 ? lego_softmax_f32s_l32_launch
                  : lego_rowwise_f16_wpr(M, 2 * N) == 8 ? lego_softmax_f32s_w8_launch
                  : long_row ? lego_softmax_f32s_w16_launch : N <= 1024 ? lego_softmax_f32s_w1_launch
                                                                      : lego_softmax_f32s_w4_launch)(x, y, M, N, as_stream(stream)));
  if (N <= 1024)   // rows of at most 16 or 32 vectors: several rows per wave
    return ok_or((N <= 64 ? lego_softmax_f32_l16_launch : N <= 128 ? lego_softmax_f32_l32_launch : lego_softmax_f32_w1_launch)(
        x, y, M, N, as_stream(stream)));
  // eight waves for the rows that take them in the 16-bit types, by their bytes (8192^2: softmax +3 %, LayerNorm +6 %;
  // 16384 x 4096 +6 % and +2 %)
  if (lego_rowwise_f16_wpr(M, 2 * N) == 8) return ok_or(lego_softmax_f32_w8_launch(x, y, M, N, as_stream(stream)));
  return ok_or((long_row ? lego_softmax_f32_w16_launch : lego_softmax_f32_w4_launch)(x, y, M, N, as_stream(stream)));
}

int lego_hip_layernorm_fwd_f16_wpr(const void* x, void* y, const void* w, const void* b,
                                   float* mean, float* rstd, int M, int N, float eps,
                                   int waves_per_row, void* stream)
{
  if (!usable(x) || !usable(y) || !usable(w) || !usable(b) || mean == nullptr || rstd == nullptr) return kInvalid;
  if (M <= 0 || N <= 0 || N % 8 || N > LEGO_ROWWISE_MAX_N || !(eps >= 0.0f)) return kInvalid;
  switch (waves_per_row) {
    case 1:   // rows of at most 16 or 32 vectors: several rows per wave
      return ok_or((N <= 128 ? lego_layernorm_fwd_f16_l16_launch : N <= 256 ? lego_layernorm_fwd_f16_l32_launch
                                                                         : lego_layernorm_fwd_f16_w1_launch)(
          x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
    case 2: return ok_or(lego_layernorm_fwd_f16_w2_launch(x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
    case 4: return ok_or(lego_layernorm_fwd_f16_w4_launch(x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
    case 8: return ok_or(lego_layernorm_fwd_f16_w8_launch(x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
    case 16: return ok_or(lego_layernorm_fwd_f16_w16_launch(x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
    default: return kInvalid;
  }
}

int lego_hip_layernorm_fwd_f16(const void* x, void* y, const void* w, const void* b,
                               float* mean, float* rstd, int M, int N, float eps, void* stream)
{
  if (!element_aligned(x, 2) || !element_aligned(y, 2) || !element_aligned(w, 2) || !element_aligned(b, 2)) return kInvalid;
  if (!element_aligned(mean, 4) || !element_aligned(rstd, 4)) return kInvalid;
  if (M <= 0 || N <= 0 || N > LEGO_ROWWISE_MAX_N || !(eps >= 0.0f)) return kInvalid;
  const bool long_row = N > LEGO_ROWWISE_MAX_N_SMALL_TEAMS;
  if (N % 8 || !aligned16(x) || !aligned16(y) || !aligned16(w) || !aligned16(b))   // rows of any length, or at any element
    return ok_or((N <= 128 ? lego_layernorm_fwd_f16s_l16_launch : N <= 256 ? lego_layernorm_fwd_f16s_l32_launch
                  : lego_rowwise_f16_wpr(M, N) == 8 ? lego_layernorm_fwd_f16s_w8_launch
                  : long_row ? lego_layernorm_fwd_f16s_w16_launch : lego_rowwise_default_wpr(N) == 1 ? lego_layernorm_fwd_f16s_w1_launch
                                                                                                 : lego_layernorm_fwd_f16s_w4_launch)(
        x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
  return lego_hip_layernorm_fwd_f16_wpr(x, y, w, b, mean, rstd, M, N, eps, lego_rowwise_f16_wpr(M, N), stream);
}

int lego_hip_layernorm_fwd_f32(const void* x, void* y, const void* w, const void* b,
                               float* mean, float* rstd, int M, int N, float eps, void* stream)
{
  if (!element_aligned(x, 4) || !element_aligned(y, 4) || !element_aligned(w, 4) || !element_aligned(b, 4)) return kInvalid;
  if (!element_aligned(mean, 4) || !element_aligned(rstd, 4)) return kInvalid;
  if (M <= 0 || N <= 0 || N > LEGO_ROWWISE_MAX_N || !(eps >= 0.0f)) return kInvalid;
  const bool long_row = N > LEGO_ROWWISE_MAX_N_SMALL_TEAMS;
  if (N % 4 || !aligned16(x) || !aligned16(y) || !aligned16(w) || !aligned16(b))   // rows of any length, or at any element
    return ok_or((N <= 64 ? lego_layernorm_fwd_f32s_l16_launch : N <= 128 ? lego_layernorm_fwd_f32s_l32_launch
                  : lego_rowwise_f16_wpr(M, 2 * N) == 8 ? lego_layernorm_fwd_f32s_w8_launch
                  : long_row ? lego_layernorm_fwd_f32s_w16_launch : N <= 1024 ? lego_layernorm_fwd_f32s_w1_launch
                                                                            : lego_layernorm_fwd_f32s_w4_launch)(
        x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
  if (N <= 1024)
    return ok_or((N <= 64 ? lego_layernorm_fwd_f32_l16_launch : N <= 128 ? lego_layernorm_fwd_f32_l32_launch
                                                                      : lego_layernorm_fwd_f32_w1_launch)(
        x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
  if (lego_rowwise_f16_wpr(M, 2 * N) == 8)   // as the 16-bit types, by the bytes of a row
    return ok_or(lego_layernorm_fwd_f32_w8_launch(x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
  return ok_or((long_row ? lego_layernorm_fwd_f32_w16_launch : lego_layernorm_fwd_f32_w4_launch)(
      x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
}

int lego_hip_softmax_bf16(const void* x, void* y, int M, int N, void* stream)
{
  if (!element_aligned(x, 2) || !element_aligned(y, 2) || M <= 0 || N <= 0) return kInvalid;
  if (N > LEGO_ROWWISE_MAX_N) return ok_or(lego_softmax_long_bf16_launch(x, y, M, N, as_stream(stream)));   // two passes
  const int wpr = lego_rowwise_default_wpr(N);
  if (N % 8 || !aligned16(x) || !aligned16(y))   // rows of any length, or at any element
    return ok_or((N <= 128 ? lego_softmax_bf16s_l16_launch : N <= 256 ? lego_softmax_bf16s_l32_launch
                  : lego_rowwise_f16_wpr(M, N) == 8 ? lego_softmax_bf16s_w8_launch
                  : wpr == 16 ? lego_softmax_bf16s_w16_launch : wpr == 1 ? lego_softmax_bf16s_w1_launch
                                                                       : lego_softmax_bf16s_w4_launch)(x, y, M, N, as_stream(stream)));
  if (N <= 256) return ok_or((N <= 128 ? lego_softmax_bf16_l16_launch : lego_softmax_bf16_l32_launch)(x, y, M, N, as_stream(stream)));
  if (lego_rowwise_f16_wpr(M, N) == 8) return ok_or(lego_softmax_bf16_w8_launch(x, y, M, N, as_stream(stream)));   // as fp16
  return ok_or((wpr == 16 ? lego_softmax_bf16_w16_launch : wpr == 1 ? lego_softmax_bf16_w1_launch
                                                                    : lego_softmax_bf16_w4_launch)(x, y, M, N, as_stream(stream)));
}

int lego_hip_layernorm_fwd_bf16(const void* x, void* y, const void* w, const void* b,
                                float* mean, float* rstd, int M, int N, float eps, void* stream)
{
  if (!element_aligned(x, 2) || !element_aligned(y, 2) || !element_aligned(w, 2) || !element_aligned(b, 2)) return kInvalid;
  if (!element_aligned(mean, 4) || !element_aligned(rstd, 4)) return kInvalid;
  if (M <= 0 || N <= 0 || N > LEGO_ROWWISE_MAX_N || !(eps >= 0.0f)) return kInvalid;
  const int wpr = lego_rowwise_default_wpr(N);
  if (N % 8 || !aligned16(x) || !aligned16(y) || !aligned16(w) || !aligned16(b))   // rows of any length, or at any element
    return ok_or((N <= 128 ? lego_layernorm_fwd_bf16s_l16_launch : N <= 256 ? lego_layernorm_fwd_bf16s_l32_launch
                  : lego_rowwise_f16_wpr(M, N) == 8 ? lego_layernorm_fwd_bf16s_w8_launch
                  : wpr == 16 ? lego_layernorm_fwd_bf16s_w16_launch : wpr == 1 ? lego_layernorm_fwd_bf16s_w1_launch
                                                                             : lego_layernorm_fwd_bf16s_w4_launch)(
        x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
  if (N <= 256)
    return ok_or((N <= 128 ? lego_layernorm_fwd_bf16_l16_launch : lego_layernorm_fwd_bf16_l32_launch)(
        x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
  if (lego_rowwise_f16_wpr(M, N) == 8)   // as fp16
    return ok_or(lego_layernorm_fwd_bf16_w8_launch(x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
  return ok_or((wpr == 16 ? lego_layernorm_fwd_bf16_w16_launch : wpr == 1 ? lego_layernorm_fwd_bf16_w1_launch
                                                                          : lego_layernorm_fwd_bf16_w4_launch)(
      x, y, w, b, mean, rstd, M, N, eps, as_stream(stream)));
}

int lego_hip_layernorm_bwd_workspace_bytes(int M, int N, unsigned long long* bytes)
{
  if (bytes == nullptr || M <= 0 || N <= 0 || N > LEGO_LAYERNORM_BWD_MAX_N) return kInvalid;
  const unsigned long long pitch = (static_cast<unsigned long long>(N) + 7) / 8 * 8;
  *bytes = 2ull * lego_layernorm_bwd_groups(M, N) * pitch * sizeof(float);
  return 0;
}

int lego_hip_layernorm_bwd_f16(const void* dy, const void* x, const void* w, const float* mean,
                               const float* rstd, void* dx, void* dw, void* db, void* workspace,
                               unsigned long long workspace_bytes, int M, int N, void* stream)
{
  unsigned long long need = 0;
  if (lego_hip_layernorm_bwd_workspace_bytes(M, N, &need) != 0) return kInvalid;
  if (!element_aligned(dy, 2) || !element_aligned(x, 2) || !element_aligned(w, 2) || !element_aligned(dx, 2) ||
      !element_aligned(dw, 2) || !element_aligned(db, 2) || !usable(workspace))
    return kInvalid;
  if (!element_aligned(mean, 4) || !element_aligned(rstd, 4) || workspace_bytes < need) return kInvalid;
  const int any_base = !(aligned16(dy) && aligned16(x) && aligned16(w) && aligned16(dx));
  return ok_or(lego_layernorm_bwd_f16_launch(dy, x, w, mean, rstd, dx, dw, db, static_cast<float*>(workspace), M, N, any_base,
                                             as_stream(stream)));
}

int lego_hip_layernorm_bwd_f16_noalloc(const void* dy, const void* x, const void* w, const float* mean,
                                       const float* rstd, void* dx, void* dw, void* db, int M, int N, void* stream)
{
  unsigned long long need = 0;
  if (lego_hip_layernorm_bwd_workspace_bytes(M, N, &need) != 0) return kInvalid;
  if (need > kScratchBytes) return kInvalid;     // partial rows beyond the built-in scratch
  if (!element_aligned(dy, 2) || !element_aligned(x, 2) || !element_aligned(w, 2) || !element_aligned(dx, 2) ||
      !element_aligned(dw, 2) || !element_aligned(db, 2))
    return kInvalid;
  if (!element_aligned(mean, 4) || !element_aligned(rstd, 4)) return kInvalid;
  const int any_base = !(aligned16(dy) && aligned16(x) && aligned16(w) && aligned16(dx));
  float* partials = nullptr;
  const hipError_t err = scratch_address(&partials);
  if (err != hipSuccess) return ok_or(err);
  // every partial row that the reduction reads is written by the first stage of the same call, so
  // what an earlier call left in the array needs no clearing
  return ok_or(lego_layernorm_bwd_f16_launch(dy, x, w, mean, rstd, dx, dw, db, partials, M, N, any_base, as_stream(stream)));
}

int lego_hip_layernorm_bwd_f32_workspace_bytes(int M, int N, unsigned long long* bytes)
{
  if (bytes == nullptr || M <= 0 || N <= 0 || N > LEGO_LAYERNORM_BWD_MAX_N) return kInvalid;
  const unsigned long long pitch = (static_cast<unsigned long long>(N) + 7) / 8 * 8;
  *bytes = 2ull * lego_layernorm_bwd_f32_groups(M, N) * pitch * sizeof(float);
  return 0;
}

int lego_hip_layernorm_bwd_f32(const void* dy, const void* x, const void* w, const float* mean,
                               const float* rstd, void* dx, void* dw, void* db, void* workspace,
                               unsigned long long workspace_bytes, int M, int N, void* stream)
{
  unsigned long long need = 0;
  if (lego_hip_layernorm_bwd_f32_workspace_bytes(M, N, &need) != 0) return kInvalid;
  if (!element_aligned(dy, 4) || !element_aligned(x, 4) || !element_aligned(w, 4) || !element_aligned(dx, 4) ||
      !element_aligned(dw, 4) || !element_aligned(db, 4) || !usable(workspace))
    return kInvalid;
  if (!element_aligned(mean, 4) || !element_aligned(rstd, 4) || workspace_bytes < need) return kInvalid;
  const int any_base = !(aligned16(dy) && aligned16(x) && aligned16(w) && aligned16(dx));
  return ok_or(lego_layernorm_bwd_f32_launch(dy, x, w, mean, rstd, dx, dw, db, static_cast<float*>(workspace), M, N, any_base,
                                             as_stream(stream)));
}

int lego_hip_layernorm_bwd_bf16_workspace_bytes(int M, int N, unsigned long long* bytes)
{
  if (bytes == nullptr || M <= 0 || N <= 0 || N > LEGO_LAYERNORM_BWD_MAX_N) return kInvalid;
  const unsigned long long pitch = (static_cast<unsigned long long>(N) + 7) / 8 * 8;
  *bytes = 2ull * lego_layernorm_bwd_bf16_groups(M, N) * pitch * sizeof(float);
  return 0;
}

int lego_hip_layernorm_bwd_bf16(const void* dy, const void* x, const void* w, const float* mean,
                                const float* rstd, void* dx, void* dw, void* db, void* workspace,
                                unsigned long long workspace_bytes, int M, int N, void* stream)
{
  unsigned long long need = 0;
  if (lego_hip_layernorm_bwd_bf16_workspace_bytes(M, N, &need) != 0) return kInvalid;
  if (!element_aligned(dy, 2) || !element_aligned(x, 2) || !element_aligned(w, 2) || !element_aligned(dx, 2) ||
      !element_aligned(dw, 2) || !element_aligned(db, 2) || !usable(workspace))
    return kInvalid;
  if (!element_aligned(mean, 4) || !element_aligned(rstd, 4) || workspace_bytes < need) return kInvalid;
  const int any_base = !(aligned16(dy) && aligned16(x) && aligned16(w) && aligned16(dx));
  return ok_or(lego_layernorm_bwd_bf16_launch(dy, x, w, mean, rstd, dx, dw, db, static_cast<float*>(workspace), M, N, any_base,
                                              as_stream(stream)));
}

namespace {
typedef hipError_t (*gemm_launcher)(const void*, const void*, void*, int, int, int, int, hipStream_t);
struct GemmKernels {
  gemm_launcher big[4];     // 256 x 256 tiles, one workgroup per CU; index 2*trans_a + trans_b
  gemm_launcher small[4];   // 128 x 128 tiles, two workgroups per CU (null: not built for this type)
  gemm_launcher sparse[4];  // 256 x 256 tiles on 32x32x16 MFMAs, for launches that leave many CUs idle (null: not built for this type)
};
// Fewer 256 x 256 tiles than this and the 128 x 128 kernel, with four times as many workgroups,
// keeps more of the 256 CUs busy than its higher LDS traffic per flop costs.
constexpr long kSmallTileBelow = 129;
// One round of 256 x 256 tiles that leaves this many CUs or more without a tile runs faster on the 32x32x16 MFMA: away
// from the socket's power limit its fewer LDS reads per flop count for more than the 16x16x32's lower energy per flop
// (fp16, 144 tiles: 0.95 -> 1.02 PFLOP/s at 2304 x 4096 x 4096, 0.75 -> 0.85 at 3072 x 3072 x 1024; 160 tiles 1.05 -> 1.08;
// 176 tiles 1.08 -> 1.09; 192 tiles 1.16 -> 1.14).
constexpr long kSparseRoundBelow = 176;
// Time of a last round in which only `share` of the workgroup slots hold a tile, in units of a full round.  A few busy
// CUs run at the clock that the socket's power limit denies the full chip, so the round is shorter than a full one
// even though each of its tiles takes a CU to itself.
inline double partial_round(double share, double least, double knee)
{
  if (share <= 0.0) return 0.0;
  return share <= knee ? least : least + (share - knee) * (1.0 - least) / (1.0 - knee);
}
// Larger products whose 256 x 256 tiles leave the last round of workgroups mostly empty take the small tile when the
// estimate of its time is the lower one: whole rounds of 256 big or 512 small tiles (the small tile runs at about 0.8
// of the large tile's rate, so a round of it costs 0.625 of a big one) plus the partial last round.  Measured on fp16
// products 4096 deep, time of a round of big tiles by the share of CUs it keeps busy: 0.06-0.5 -> 0.69-0.71, 0.56 ->
// 0.76, 0.69 -> 0.82, 0.81 -> 0.88, 0.94 -> 0.97; of small tiles: 0.13 -> 0.51, 0.5 -> 0.58.  4352 x 4096 x 4096 (272
// tiles): 0.81 big, 0.87 small; 5120 x 4096 (320): 0.95 / 1.00; 4608^3 (324): 0.98 / 1.02; 6144 x 4096 (384, a half
// round left over): 1.13 / 1.04; 5120^3 and 6144^3 stay with the big tile.
inline bool small_tiles_fill_better(int M, int N, long tiles)
{
  if (tiles < kSmallTileBelow) return true;
  const long small = static_cast<long>((M + 127) / 128) * ((N + 127) / 128);
  const double big_time = static_cast<double>(tiles / 256) + partial_round(static_cast<double>(tiles % 256) / 256.0, 0.69, 0.5);
  const double small_time = 0.625 * (static_cast<double>(small / 512) + partial_round(static_cast<double>(small % 512) / 512.0, 0.5, 0.4));
  return small_time < big_time;
}

// Which build a product in whole 16-byte chunks takes: 0 = 256 x 256 tiles on the type's own MFMA, 1 = 128 x 128 tiles,
// 2 = 256 x 256 tiles on the 32x32x16 MFMA (16-bit operands: one round that leaves a third of the CUs idle).
inline int gemm_choice(int M, int N, bool has_small, bool has_sparse)
{
  const long tiles = static_cast<long>((M + LEGO_GEMM_BM - 1) / LEGO_GEMM_BM) * ((N + LEGO_GEMM_BN - 1) / LEGO_GEMM_BN);
  if (has_small && small_tiles_fill_better(M, N, tiles)) return 1;
  return has_sparse && tiles < kSparseRoundBelow ? 2 : 0;
}

int gemm_ex(const GemmKernels& k, int element, const void* a, const void* b, void* c, int M, int N, int K,
            int trans_a, int trans_b, int activation, void* stream, int bk = LEGO_GEMM_BK, int chunk = 8)
{
  if (a == nullptr || b == nullptr || c == nullptr || M <= 0 || N <= 0 || K <= 0) return kInvalid;
  if (activation != 0 && activation != 1) return kInvalid;
  // The tiled kernels move 16-byte chunks (`chunk` elements): bases 16-byte aligned and every operand row
  // in whole chunks -- rows of C and of B as given run along N, rows of A as given and of a transposed B
  // along K, rows of a transposed A along M.  Tiles may be ragged in M, N and K.  Everything else -- the
  // reference keeps M, N, K symbolic (matmul_sympy.py:69-70) -- goes to the kernel that moves one element
  // per access.
  (void)bk;
  const bool tiled = usable(a) && usable(b) && usable(c) && N % chunk == 0 &&
                     (trans_a ? M % chunk == 0 : K % chunk == 0) && (!trans_b || K % chunk == 0);
  if (!tiled) {
    const uintptr_t in_mask = element <= 1 || element == 4 ? 1u : 0u;       // 2-byte or 1-byte operand elements; C is 2-byte
    if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & in_mask) return kInvalid;
    if (reinterpret_cast<uintptr_t>(c) & 1u) return kInvalid;
    return ok_or(lego_gemm_any_launch(a, b, c, M, N, K, trans_a ? 1 : 0, trans_b ? 1 : 0, activation, element,
                                      as_stream(stream)));
  }
  const int layout = (trans_a ? 2 : 0) + (trans_b ? 1 : 0);
  const int choice = gemm_choice(M, N, k.small[layout] != nullptr, k.sparse[layout] != nullptr);
  const gemm_launcher* by_layout = choice == 1 ? k.small : choice == 2 ? k.sparse : k.big;
  return ok_or(by_layout[layout](a, b, c, M, N, K, activation, as_stream(stream)));
}

// Parts along K for a product of few tiles (1: one workgroup per tile does it all): enough parts for two
// workgroups of 128 x 128 tiles per CU, at least four k-tiles each.  The second launch and the partial sums cost
// about what 16 k-tiles take, so shallower products stay whole (1024^3: 8.6 us whole, 11.7 in four parts;
// 512 x 512 x 2048: 13.7 whole, 8.2 in eight).
int splitk_parts(int M, int N, int K, int bk)
{
  const long tiles = static_cast<long>((M + 127) / 128) * ((N + 127) / 128), depth = (K + bk - 1) / bk;
  if (tiles > 128 || depth < 32) return 1;
  long parts = (512 + tiles - 1) / tiles;
  if (parts > depth / 4) parts = depth / 4;
  if (parts > 64) parts = 64;
  return parts < 2 ? 1 : static_cast<int>(parts);
}
typedef hipError_t (*splitk_launcher)(const void*, const void*, void*, int, int, int, int, int, float*, hipStream_t);

// 8-bit operands: the small tile only where both operands are k-major (A as given, B transposed)
#define LEGO_GEMM_KERNELS_SMALL_NT(DT)                                                                 \
  {{lego_gemm_##DT##_nn_launch, lego_gemm_##DT##_nt_launch, lego_gemm_##DT##_tn_launch,              \
    lego_gemm_##DT##_tt_launch},                                                                       \
   {nullptr, lego_gemm_##DT##_nt_t128x128_launch, nullptr, nullptr}}
#define LEGO_GEMM_KERNELS(DT)                                                                          \
  {{lego_gemm_##DT##_nn_launch, lego_gemm_##DT##_nt_launch, lego_gemm_##DT##_tn_launch,              \
    lego_gemm_##DT##_tt_launch},                                                                       \
   {lego_gemm_##DT##_nn_t128x128_launch, lego_gemm_##DT##_nt_t128x128_launch,                         \
    lego_gemm_##DT##_tn_t128x128_launch, lego_gemm_##DT##_tt_t128x128_launch},                         \
   {lego_gemm_##DT##_nn_m32_launch, lego_gemm_##DT##_nt_m32_launch, lego_gemm_##DT##_tn_m32_launch,  \
    lego_gemm_##DT##_tt_m32_launch}}
}  // namespace

int lego_hip_gemm_f16_ex(const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                         int activation, void* stream)
{
  static const GemmKernels k = LEGO_GEMM_KERNELS(f16);
  return gemm_ex(k, 0, a, b, c, M, N, K, trans_a, trans_b, activation, stream);
}

int lego_hip_gemm_bf16_ex(const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                          int activation, void* stream)
{
  static const GemmKernels k = LEGO_GEMM_KERNELS(bf16);
  return gemm_ex(k, 1, a, b, c, M, N, K, trans_a, trans_b, activation, stream);
}

int lego_hip_gemm_bf16_f16_ex(const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                              int activation, void* stream)
{
  static const GemmKernels k = LEGO_GEMM_KERNELS(bf16h);
  return gemm_ex(k, 4, a, b, c, M, N, K, trans_a, trans_b, activation, stream);
}

int lego_hip_gemm_workspace_bytes(int M, int N, int K, unsigned long long* bytes)
{
  if (bytes == nullptr || M <= 0 || N <= 0 || K <= 0) return kInvalid;
  // N or K not a multiple of 8: room for zero-padded copies of both operands and of the result (2-byte elements).
  // (M only matters as the row length of a transposed A; that case alone stays with the one-element kernel.)
  unsigned long long copies = 0;
  if (N % 8 || K % 8) {
    const unsigned long long m8 = (M + 7ull) / 8 * 8, n8 = (N + 7ull) / 8 * 8, k8 = (K + 7ull) / 8 * 8;
    copies = 2ull * (m8 * k8 + k8 * n8 + m8 * n8);
    M = static_cast<int>(m8); N = static_cast<int>(n8); K = static_cast<int>(k8);     // the product that then runs
  }
  const int parts = splitk_parts(M, N, K, LEGO_GEMM_BK);
  const unsigned long long tiles = static_cast<unsigned long long>((M + 127) / 128) * ((N + 127) / 128);
  *bytes = copies + (parts > 1 ? parts * tiles * 128ull * 128ull * sizeof(float) : 0ull);
  return 0;
}

int lego_hip_gemm_ex_ws(int element, const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                        int activation, void* workspace, unsigned long long workspace_bytes, void* stream)
{
#define LEGO_SPLITK(DT) {lego_gemm_##DT##_nn_t128x128_splitk_launch, lego_gemm_##DT##_nt_t128x128_splitk_launch, \
                         lego_gemm_##DT##_tn_t128x128_splitk_launch, lego_gemm_##DT##_tt_t128x128_splitk_launch}
  static const splitk_launcher f16[4] = LEGO_SPLITK(f16), bf16[4] = LEGO_SPLITK(bf16), bf16h[4] = LEGO_SPLITK(bf16h);
#undef LEGO_SPLITK
  if (element != 0 && element != 1 && element != 4) return kInvalid;
  unsigned long long need = 0;
  if (lego_hip_gemm_workspace_bytes(M, N, K, &need) != 0) return kInvalid;
  // what the tiled kernels ask of shapes and bases (gemm_ex): anything else, and every product that gains nothing
  // from parts, takes the plain entry point
  const bool tiled = usable(a) && usable(b) && usable(c) && N % 8 == 0 && (trans_a ? M % 8 == 0 : K % 8 == 0) &&
                     (!trans_b || K % 8 == 0);
  const bool have_workspace = need != 0 && workspace != nullptr && workspace_bytes >= need && usable(workspace);
  if (have_workspace && (N % 8 || K % 8)) {
    // Operand rows that are not whole 16-byte chunks: the tiled kernels run on zero-padded copies (every side a
    // multiple of 8; the padding adds zeros to the sums) and the result is copied back.  Three more passes over
    // the matrices, against the tenfold cost of the kernel that moves one element per access.
    if (a == nullptr || b == nullptr || c == nullptr || (activation != 0 && activation != 1)) return kInvalid;
    if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 1u) return kInvalid;
    const int M8 = (M + 7) / 8 * 8, N8 = (N + 7) / 8 * 8, K8 = (K + 7) / 8 * 8;
    const int Mp = trans_a ? M8 : M;                 // rows of the padded product: a transposed A has rows of M elements
    uint16_t* ap = static_cast<uint16_t*>(workspace);
    uint16_t* bp = ap + static_cast<size_t>(M8) * K8;
    uint16_t* cp = bp + static_cast<size_t>(K8) * N8;
    const bool copy_a = K8 != K || (trans_a && M8 != M) || !usable(a);
    const bool copy_b = K8 != K || N8 != N || !usable(b);
    const bool copy_c = N8 != N || Mp != M || !usable(c);
    hipError_t err = hipSuccess;
    if (copy_a) err = trans_a ? pad2d(a, ap, K, M, K8, M8, as_stream(stream)) : pad2d(a, ap, M, K, M, K8, as_stream(stream));
    if (err != hipSuccess) return ok_or(err);
    if (copy_b) err = trans_b ? pad2d(b, bp, N, K, N8, K8, as_stream(stream)) : pad2d(b, bp, K, N, K8, N8, as_stream(stream));
    if (err != hipSuccess) return ok_or(err);
    const void* aa = copy_a ? ap : a;
    const void* bb = copy_b ? bp : b;
    void* cc = copy_c ? cp : c;
    int rc;
    const int parts = splitk_parts(Mp, N8, K8, LEGO_GEMM_BK);
    if (parts > 1) {      // few tiles: parts along K, their sums behind the copies (the size asked for covers M8 rows)
      const splitk_launcher* by_layout = element == 0 ? f16 : element == 1 ? bf16 : bf16h;
      rc = ok_or(by_layout[(trans_a ? 2 : 0) + (trans_b ? 1 : 0)](aa, bb, cc, Mp, N8, K8, activation, parts,
                                                                 reinterpret_cast<float*>(cp + static_cast<size_t>(M8) * N8),
                                                                 as_stream(stream)));
    } else {
      switch (element) {
        case 0: rc = lego_hip_gemm_f16_ex(aa, bb, cc, Mp, N8, K8, trans_a, trans_b, activation, stream); break;
        case 1: rc = lego_hip_gemm_bf16_ex(aa, bb, cc, Mp, N8, K8, trans_a, trans_b, activation, stream); break;
        default: rc = lego_hip_gemm_bf16_f16_ex(aa, bb, cc, Mp, N8, K8, trans_a, trans_b, activation, stream); break;
      }
    }
    if (rc != 0 || !copy_c) return rc;
    return ok_or(unpad2d(cp, c, M, N, N8, as_stream(stream)));
  }
  if (!have_workspace || !tiled) {
    switch (element) {
      case 0: return lego_hip_gemm_f16_ex(a, b, c, M, N, K, trans_a, trans_b, activation, stream);
      case 1: return lego_hip_gemm_bf16_ex(a, b, c, M, N, K, trans_a, trans_b, activation, stream);
      default: return lego_hip_gemm_bf16_f16_ex(a, b, c, M, N, K, trans_a, trans_b, activation, stream);
    }
  }
  if (a == nullptr || b == nullptr || c == nullptr || (activation != 0 && activation != 1)) return kInvalid;
  const splitk_launcher* by_layout = element == 0 ? f16 : element == 1 ? bf16 : bf16h;
  return ok_or(by_layout[(trans_a ? 2 : 0) + (trans_b ? 1 : 0)](a, b, c, M, N, K, activation, splitk_parts(M, N, K, LEGO_GEMM_BK),
                                                             static_cast<float*>(workspace), as_stream(stream)));
}

int lego_hip_gemm_fp8_ex(const void* a, const void* b, void* c, int M, int N, int K, int trans_a, int trans_b,
                         int activation, int format, void* stream)
{
  static const GemmKernels e4m3 = LEGO_GEMM_KERNELS_SMALL_NT(e4m3);
  static const GemmKernels e5m2 = LEGO_GEMM_KERNELS_SMALL_NT(e5m2);
  if (format != 0 && format != 1) return kInvalid;
  return gemm_ex(format == 0 ? e4m3 : e5m2, format == 0 ? 2 : 3, a, b, c, M, N, K, trans_a, trans_b, activation,
                 stream, LEGO_GEMM_BK_8BIT, 16);
}

int lego_hip_gemm_f16_variant(const void* a, const void* b, void* c, int M, int N, int K, int variant, void* stream)
{
  if (!usable(a) || !usable(b) || !usable(c) || M <= 0 || N <= 0 || K <= 0 || N % 8 || K % 8) return kInvalid;
  if (variant == 0) return ok_or(lego_gemm_f16_nn_launch(a, b, c, M, N, K, 0, as_stream(stream)));
  if (variant == 1) return ok_or(lego_gemm_f16_nn_m32_launch(a, b, c, M, N, K, 0, as_stream(stream)));
  if (variant == 2) return ok_or(lego_gemm_f16_nn_w2x4_launch(a, b, c, M, N, K, 0, as_stream(stream)));
  if (variant == 3) return ok_or(lego_gemm_f16_nn_stamps_launch(a, b, c, M, N, K, 0, as_stream(stream)));
  return kInvalid;
}

int lego_hip_gemm_f16_act(const void* a, const void* b, void* c, int M, int N, int K, int activation, void* stream)
{
  return lego_hip_gemm_f16_ex(a, b, c, M, N, K, 0, 0, activation, stream);
}

int lego_hip_gemm_f16(const void* a, const void* b, void* c, int M, int N, int K, void* stream)
{
  return lego_hip_gemm_f16_ex(a, b, c, M, N, K, 0, 0, 0, stream);
}

namespace {
int stencil(const float* in, float* out, const float* c, int n, int radius, int kind, int bricks, void* stream)
{
  if (!usable(in) || !usable(out) || c == nullptr || in == out) return kInvalid;
  if (n <= 0 || n % LEGO_STENCIL_BRICK || n > 1024 || radius < 1 || radius > (kind == 1 ? LEGO_STENCIL_STAR_MAX_RADIUS : LEGO_STENCIL_MAX_RADIUS) || 2 * radius >= n)
    return kInvalid;
  return ok_or(lego_stencil_f32_launch(in, out, c, n, radius, kind, bricks ? 1 : 0, as_stream(stream)));
}
}  // namespace

int lego_hip_stencil_f3d_f32(const float* in, float* out, const float* c, int n, int radius, int bricks, void* stream)
{
  return stencil(in, out, c, n, radius, 0, bricks, stream);
}

int lego_hip_stencil_laplacian_f32(const float* in, float* out, const float* c, int n, int radius, int bricks,
                                   void* stream)
{
  return stencil(in, out, c, n, radius, 1, bricks, stream);
}

int lego_hip_lud_f32(float* m, int n, void* stream)
{
  if (!usable(m)) return kInvalid;
  if (n <= 0 || n % LEGO_LUD_BLOCK || n > 32768) return kInvalid;
  return ok_or(lego_lud_f32_launch(m, n, as_stream(stream)));
}

int lego_hip_lud_f32_plan(int n, int* records, int capacity, int* count)
{
  if (!count || capacity < 0 || (capacity > 0 && !records)) return kInvalid;
  if (n <= 0 || n % LEGO_LUD_BLOCK || n > 32768) return kInvalid;
  return ok_or(lego_lud_f32_plan(n, records, capacity, count));
}

int lego_hip_nw_i32(const int* reference, int* matrix, int n, int penalty, void* stream)
{
  if (!usable(reference) || !usable(matrix)) return kInvalid;
  if (n <= 0 || n % LEGO_NW_TILE || n > 32768) return kInvalid;
  return ok_or(lego_nw_i32_launch(reference, matrix, n, penalty, as_stream(stream)));
}

namespace {
// Time of a grouped launch: list scheduling of its workgroups, in launch order, on `slots` workgroups
// that run at once (a workgroup goes to the slot that frees up first).  The launch is a sequence of
// batches of count[i] workgroups that take cost[i] each.  The slot loads are kept as a sorted list of
// (load, how many slots) levels, so a batch of equal workgroups costs a few steps.
double grouped_makespan(const long* count, const double* cost, int batches, long slots)
{
  struct Level { double load; long count; };
  Level lv[8 * LEGO_GROUPED_MAX_GROUPS + 8];
  int n = 1;
  lv[0] = {0.0, slots};
  for (int g = 0; g < batches; ++g) {
    long left = count[g];
    const double d = cost[g];
    while (left > 0) {
      // the least loaded level takes workgroups, one per slot; its slots move up by d
      const long take = left < lv[0].count ? left : lv[0].count;
      const double moved = lv[0].load + d;
      lv[0].count -= take;
      left -= take;
      if (lv[0].count == 0) {
        for (int i = 1; i < n; ++i) lv[i - 1] = lv[i];
        --n;
      }
      // insert (moved, take) keeping the list sorted; merge equal loads
      int pos = 0;
      while (pos < n && lv[pos].load < moved) ++pos;
      if (pos < n && lv[pos].load == moved) {
        lv[pos].count += take;
      } else if (n < static_cast<int>(sizeof(lv) / sizeof(lv[0]))) {
        for (int i = n; i > pos; --i) lv[i] = lv[i - 1];
        lv[pos] = {moved, take};
        ++n;
      } else {
        lv[n - 1].count += take;        // out of levels (never with <= 64 groups): fold into the top one
        if (lv[n - 1].load < moved) lv[n - 1].load = moved;
      }
    }
  }
  return lv[n - 1].load;
}

// What a grouped call launches: the kernel on 256 x 256 tiles with the last `split` tiles of its launch
// order as two 128 x 256 halves each (kind 0), or the kernel on 128 x 128 tiles (kind 1).
struct GroupedPlan {
  int kind, tiles, split;
};

// Costs in units of one k-tile step of a 256 x 256 tile that has its CU to itself (about 1.8 us for
// fp16), measured on MI355X: a tile pays a start-up and an epilogue on top of its steps (31.4 us for
// 16 steps); a 128 x 256 half-tile takes 19.2 us for 16 steps; a 128 x 128 tile sharing its CU with
// another one takes 0.66 of a whole tile of the same depth.
constexpr double kTileOverhead = 1.6, kHalfStep = 0.58, kHalfOverhead = 1.5, kSmallCost = 0.66;
// Problems per call.  A launch carries its pointers and sizes as kernel arguments, LEGO_GROUPED_MAX_GROUPS problems
// at most; a call with more is enqueued as several launches (below).
constexpr int kGroupedMaxProblems = 1 << 20;

GroupedPlan grouped_plan_uncached(const int* sizes3, int groups)
{
  GroupedPlan plan;
  int order[LEGO_GROUPED_MAX_GROUPS];       // problems in launch order: decreasing depth, stable
  for (int g = 0; g < groups; ++g) order[g] = g;
  for (int i = 1; i < groups; ++i) {
    const int o = order[i];
    int j = i;
    while (j > 0 && sizes3[3 * order[j - 1] + 2] < sizes3[3 * o + 2]) { order[j] = order[j - 1]; --j; }
    order[j] = o;
  }
  long big[LEGO_GROUPED_MAX_GROUPS], small[LEGO_GROUPED_MAX_GROUPS];
  double depth[LEGO_GROUPED_MAX_GROUPS], small_cost[LEGO_GROUPED_MAX_GROUPS];
  long total = 0;
  for (int s = 0; s < groups; ++s) {
    const int g = order[s];
    const int m = sizes3[3 * g], n = sizes3[3 * g + 1];
    big[s] = static_cast<long>((m + 255) / 256) * ((n + 255) / 256);
    small[s] = static_cast<long>((m + 127) / 128) * ((n + 127) / 128);
    depth[s] = (sizes3[3 * g + 2] + LEGO_GEMM_BK - 1) / LEGO_GEMM_BK;
    small_cost[s] = kSmallCost * (depth[s] + kTileOverhead);
    total += big[s];
  }
  const long cus = 256;                 // MI355X
  // 256 x 256 tiles, the last `split` of them as halves: the best split among multiples of 16 tiles
  // up to two rounds of the CUs
  double best = 0.0;
  long best_split = 0;
  const long max_split = total < 2 * cus ? total : 2 * cus;
  for (long split = 0; split <= max_split; split += 16) {
    long count[2 * LEGO_GROUPED_MAX_GROUPS];
    double cost[2 * LEGO_GROUPED_MAX_GROUPS];
    int nb = 0;
    long whole_left = total - split;
    for (int s = 0; s < groups; ++s) {
      const long w = big[s] < whole_left ? big[s] : whole_left;
      whole_left -= w;
      if (w > 0) { count[nb] = w; cost[nb++] = depth[s] + kTileOverhead; }
    }
    whole_left = total - split;
    for (int s = 0; s < groups; ++s) {
      const long w = big[s] < whole_left ? big[s] : whole_left;
      whole_left -= w;
      if (big[s] > w) { count[nb] = 2 * (big[s] - w); cost[nb++] = kHalfStep * depth[s] + kHalfOverhead; }
    }
    const double t = grouped_makespan(count, cost, nb, cus);
    // equal estimates: the larger split (more, shorter workgroups in the last round measured faster)
    if (split == 0 || t <= best) { best = t; best_split = split; }
  }
  const double t_small = grouped_makespan(small, small_cost, groups, 2 * cus);
  plan.kind = t_small < best ? 1 : 0;
  plan.tiles = static_cast<int>(total);
  plan.split = plan.kind == 0 ? static_cast<int>(best_split) : 0;
  return plan;
}

// The plan is a few hundred list-scheduling steps per candidate split, tens of microseconds of host time in front
// of a launch of about a hundred: a serving loop calls with the same sizes again and again, so the last few plans
// are kept, keyed by the sizes themselves.
GroupedPlan grouped_plan(const int* sizes3, int groups)
{
  struct Kept { int groups; int sizes[3 * LEGO_GROUPED_MAX_GROUPS]; GroupedPlan plan; };
  constexpr int kKept = 8;
  static Kept kept[kKept];
  static int next = 0;
  static std::mutex kept_mutex;
  const size_t bytes = sizeof(int) * 3 * static_cast<size_t>(groups);
  {
    std::lock_guard<std::mutex> hold(kept_mutex);
    for (int i = 0; i < kKept; ++i)
      if (kept[i].groups == groups && memcmp(kept[i].sizes, sizes3, bytes) == 0) return kept[i].plan;
  }
  const GroupedPlan plan = grouped_plan_uncached(sizes3, groups);
  std::lock_guard<std::mutex> hold(kept_mutex);
  Kept& slot = kept[next];
  next = (next + 1) % kKept;
  slot.groups = groups;
  memcpy(slot.sizes, sizes3, bytes);
  slot.plan = plan;
  return plan;
}

// 0: every problem fits the tiled kernels (one launch); 2: the arguments are valid but some problem needs
// the element-wise kernel (N or K not in whole 16-byte chunks, a base that is not 16-byte aligned);
// kInvalid otherwise
int grouped_check(const void* const* a, const void* const* b, void* const* c, const int* sizes3, int groups)
{
  if (a == nullptr || b == nullptr || c == nullptr || sizes3 == nullptr) return kInvalid;
  if (groups <= 0 || groups > kGroupedMaxProblems) return kInvalid;
  int verdict = 0;
  for (int g = 0; g < groups; ++g) {
    const int m = sizes3[3 * g], n = sizes3[3 * g + 1], k = sizes3[3 * g + 2];
    if (a[g] == nullptr || b[g] == nullptr || c[g] == nullptr || m <= 0 || n <= 0 || k <= 0) return kInvalid;
    if ((reinterpret_cast<uintptr_t>(a[g]) | reinterpret_cast<uintptr_t>(b[g]) | reinterpret_cast<uintptr_t>(c[g])) & 1u)
      return kInvalid;
    if (!usable(a[g]) || !usable(b[g]) || !usable(c[g]) || n % 8 || k % 8) verdict = 2;    // M may be anything
  }
  return verdict;
}

// A grouped call with a problem that the one-launch kernels do not take: one launch per problem on the
// same stream, each through the plain GEMM's dispatch (the reference walks its problems in one kernel,
// grouped_gemm.py:61-116, but takes whole tiles only).
int grouped_one_by_one(const void* const* a, const void* const* b, void* const* c, const int* sizes3, int groups,
                       void* stream)
{
  for (int g = 0; g < groups; ++g) {
    const int err = lego_hip_gemm_f16_ex(a[g], b[g], c[g], sizes3[3 * g], sizes3[3 * g + 1], sizes3[3 * g + 2], 0, 0, 0, stream);
    if (err != 0) return err;
  }
  return 0;
}
}  // namespace

namespace {
// More problems than one launch carries (the reference's host function takes any number: its tables live in
// device memory, grouped_gemm.py:120-162): all problems in order of decreasing depth (stable), cut into runs of
// LEGO_GROUPED_MAX_GROUPS, one launch per run on the same stream -- so every launch still starts with its longest
// tiles, and only the last launches hold the shallow problems whose tail rounds are short.
int grouped_in_runs(const void* const* a, const void* const* b, void* const* c, const int* sizes3, int groups, void* stream)
{
  std::vector<int> order(static_cast<size_t>(groups));
  for (int g = 0; g < groups; ++g) order[static_cast<size_t>(g)] = g;
  std::stable_sort(order.begin(), order.end(), [sizes3](int p, int q) { return sizes3[3 * p + 2] > sizes3[3 * q + 2]; });
  const void* ra[LEGO_GROUPED_MAX_GROUPS];
  const void* rb[LEGO_GROUPED_MAX_GROUPS];
  void* rc[LEGO_GROUPED_MAX_GROUPS];
  int rs[3 * LEGO_GROUPED_MAX_GROUPS];
  for (int first = 0; first < groups; first += LEGO_GROUPED_MAX_GROUPS) {
    const int count = groups - first < LEGO_GROUPED_MAX_GROUPS ? groups - first : LEGO_GROUPED_MAX_GROUPS;
    for (int i = 0; i < count; ++i) {
      const int g = order[static_cast<size_t>(first + i)];
      ra[i] = a[g]; rb[i] = b[g]; rc[i] = c[g];
      rs[3 * i] = sizes3[3 * g]; rs[3 * i + 1] = sizes3[3 * g + 1]; rs[3 * i + 2] = sizes3[3 * g + 2];
    }
    const int err = lego_hip_grouped_gemm_f16(ra, rb, rc, rs, count, stream);
    if (err != 0) return err;
  }
  return 0;
}
}  // namespace

int lego_hip_grouped_gemm_f16(const void* const* a, const void* const* b, void* const* c,
                              const int* sizes3, int groups, void* stream)
{
  const int checked = grouped_check(a, b, c, sizes3, groups);
  if (checked == 2) return grouped_one_by_one(a, b, c, sizes3, groups, stream);
  if (checked != 0) return kInvalid;
  if (groups > LEGO_GROUPED_MAX_GROUPS) return grouped_in_runs(a, b, c, sizes3, groups, stream);
  // One launch: on 256 x 256 tiles (one workgroup per CU), the last tiles of the launch order split
  // into halves when whole tiles would leave the last round mostly empty, or on 128 x 128 tiles (four
  // times as many workgroups of a quarter of the work, two per CU) when the big ones leave most CUs
  // idle; whichever the estimate finishes first.  Problems are launched in order of decreasing
  // depth, so the longest tiles start first.  (Splitting the problems over both tile sizes in two
  // launches was measured and never beat the better single launch.)
  const GroupedPlan plan = grouped_plan(sizes3, groups);
  if (plan.kind == 1) return ok_or(lego_grouped_gemm_f16_t128x128_launch(a, b, c, sizes3, groups, as_stream(stream)));
  if (plan.split == 0) return ok_or(lego_grouped_gemm_f16_launch(a, b, c, sizes3, groups, as_stream(stream)));
  return ok_or(lego_grouped_gemm_f16_split_launch(a, b, c, sizes3, groups, plan.split, as_stream(stream)));
}

int lego_hip_rows_f16_plan(int M, int N, int* waves_per_row)
{
  if (waves_per_row == nullptr || M <= 0 || N <= 0 || N % 8 != 0 || N > LEGO_ROWWISE_MAX_N) return kInvalid;
  *waves_per_row = lego_rowwise_f16_wpr(M, N);
  return 0;
}

int lego_hip_gemm_plan(int M, int N, int K, int* plan2)
{
  if (plan2 == nullptr || M <= 0 || N <= 0 || K <= 0) return kInvalid;
  const int choice = gemm_choice(M, N, true, true);
  plan2[0] = choice == 1 ? 128 : 256;
  plan2[1] = choice == 0 ? 16 : 32;
  return 0;
}

int lego_hip_grouped_gemm_f16_plan(const int* sizes3, int groups, int* plan3)
{
  if (sizes3 == nullptr || plan3 == nullptr || groups <= 0 || groups > LEGO_GROUPED_MAX_GROUPS) return kInvalid;
  for (int g = 0; g < groups; ++g)
    if (sizes3[3 * g] <= 0 || sizes3[3 * g + 1] <= 0 || sizes3[3 * g + 2] <= 0) return kInvalid;
  const GroupedPlan plan = grouped_plan(sizes3, groups);
  plan3[0] = plan.kind == 1 ? 128 : 256;
  plan3[1] = plan.tiles;
  plan3[2] = plan.split;
  return 0;
}

int lego_hip_grouped_gemm_f16_split(const void* const* a, const void* const* b, void* const* c,
                                    const int* sizes3, int groups, int split_tiles, void* stream)
{
  if (groups > LEGO_GROUPED_MAX_GROUPS || grouped_check(a, b, c, sizes3, groups) != 0) return kInvalid;     // one launch of tiled problems only
  if (split_tiles < 0)
    return ok_or(lego_grouped_gemm_f16_t128x128_launch(a, b, c, sizes3, groups, as_stream(stream)));
  return ok_or(lego_grouped_gemm_f16_split_launch(a, b, c, sizes3, groups, split_tiles, as_stream(stream)));
}

int lego_hip_grouped_gemm_f16_stamps(const void* const* a, const void* const* b, void* const* c,
                                     const int* sizes3, int groups, void* stream)
{
  if (groups > LEGO_GROUPED_MAX_GROUPS || grouped_check(a, b, c, sizes3, groups) != 0) return kInvalid;
  const GroupedPlan plan = grouped_plan(sizes3, groups);
  if (plan.kind == 1) return kInvalid;        // the measurement build exists for the 256 x 256 tiles only
  if (plan.split == 0) return ok_or(lego_grouped_gemm_f16_stamps_launch(a, b, c, sizes3, groups, as_stream(stream)));
  return ok_or(lego_grouped_gemm_f16_stamps_split_launch(a, b, c, sizes3, groups, plan.split, as_stream(stream)));
}

int lego_hip_gemm_stamps_read(unsigned long long* host, int workgroups)
{
  if (host == nullptr) return kInvalid;
  return ok_or(lego_gemm_stamps_read(host, workgroups));
}

int lego_hip_copy16(const void* in, void* out, unsigned long long bytes, void* stream)
{
  if (!usable(in) || !usable(out) || bytes == 0 || bytes % 16) return kInvalid;
  const size_t n = bytes / 16;
  const unsigned grid = static_cast<unsigned>(n / 256 < 256 * 32 ? (n + 255) / 256 : 256 * 32);
  hipLaunchKernelGGL(lego_copy16_kernel, dim3(grid), dim3(256), 0, as_stream(stream),
                     static_cast<const uint4*>(in), static_cast<uint4*>(out), n);
  return ok_or(hipGetLastError());
}

int lego_hip_copy16_stream(const void* in, void* out, unsigned long long bytes, void* stream)
{
  if (!usable(in) || !usable(out) || bytes == 0 || bytes % 16384 || bytes / 16384 > 0x7fffffffull) return kInvalid;
  hipLaunchKernelGGL(lego_copy16_stream_kernel, dim3(static_cast<unsigned>(bytes / 16384)), dim3(256), 0,
                     as_stream(stream), static_cast<const u32x4*>(in), static_cast<u32x4*>(out));
  return ok_or(hipGetLastError());
}

int lego_hip_hbm_probe(const void* in, void* out, unsigned long long bytes, int mode, int vectors_per_lane, void* stream)
{
  if (!usable(in) || !usable(out) || in == out) return kInvalid;
  if (mode < 0 || mode > 2 || (vectors_per_lane != 1 && vectors_per_lane != 4)) return kInvalid;
  const unsigned long long chunk = 4096ull * vectors_per_lane;
  if (bytes == 0 || bytes % chunk || bytes / chunk > 0x7fffffffull) return kInvalid;
  const dim3 grid(static_cast<unsigned>(bytes / chunk)), block(256);
  const u32x4* src = static_cast<const u32x4*>(in);
  u32x4* dst = static_cast<u32x4*>(out);
  hipStream_t s = as_stream(stream);
  if (vectors_per_lane == 1) {
    if (mode == 0) hipLaunchKernelGGL(lego_probe_read_kernel<1>, grid, block, 0, s, src, dst);
    else if (mode == 1) hipLaunchKernelGGL(lego_probe_write_kernel<1>, grid, block, 0, s, dst);
    else hipLaunchKernelGGL(lego_probe_copy_kernel<1>, grid, block, 0, s, src, dst);
  } else {
    if (mode == 0) hipLaunchKernelGGL(lego_probe_read_kernel<4>, grid, block, 0, s, src, dst);
    else if (mode == 1) hipLaunchKernelGGL(lego_probe_write_kernel<4>, grid, block, 0, s, dst);
    else hipLaunchKernelGGL(lego_probe_copy_kernel<4>, grid, block, 0, s, src, dst);
  }
  return ok_or(hipGetLastError());
}

int lego_hip_mfma_probe(const void* operands, float* sink, int shape, int iters, int workgroups, void* stream)
{
  if (!usable(operands) || !usable(sink) || shape < 0 || shape > 7 || iters <= 0 || workgroups <= 0) return kInvalid;
  const dim3 grid(static_cast<unsigned>(workgroups)), block(256);
  const probe_half8* src = static_cast<const probe_half8*>(operands);
  hipStream_t s = as_stream(stream);
  if (shape == 5) hipLaunchKernelGGL(lego_mfma_probe_8bit_kernel<1>, grid, block, 0, s, static_cast<const probe_int8*>(operands), sink, static_cast<unsigned>(iters));
  else if (shape == 6) hipLaunchKernelGGL(lego_mfma_probe_8bit_kernel<0>, grid, block, 0, s, static_cast<const probe_int8*>(operands), sink, static_cast<unsigned>(iters));
  else if (shape == 7) hipLaunchKernelGGL(lego_mfma_probe_8bit_16x16_kernel, grid, block, 0, s, static_cast<const probe_int8*>(operands), sink, static_cast<unsigned>(iters));
  else if (shape == 3) hipLaunchKernelGGL(lego_mfma_probe2_kernel<3>, grid, dim3(512), 0, s, src, sink, static_cast<unsigned>(iters));
  else if (shape == 4) hipLaunchKernelGGL(lego_mfma_probe2_kernel<4>, grid, dim3(512), 0, s, src, sink, static_cast<unsigned>(iters));
  else if (shape == 0) hipLaunchKernelGGL(lego_mfma_probe_kernel<0>, grid, block, 0, s, src, sink, static_cast<unsigned>(iters));
  else if (shape == 1) hipLaunchKernelGGL(lego_mfma_probe_kernel<1>, grid, block, 0, s, src, sink, static_cast<unsigned>(iters));
  else hipLaunchKernelGGL(lego_mfma_probe_kernel<2>, grid, block, 0, s, src, sink, static_cast<unsigned>(iters));
  return ok_or(hipGetLastError());
}

}  // extern "C"
