// Layout change between the network's (batch, labels, H, W) tensors and the label-innermost
// (batch, H, W, labels) layout of the message-passing kernels: a batched 2-D transpose.
//
// The reference's module does this with permute().contiguous() on the way in and out
// (pytorch/MP_module.py:199, 203, 233); the generic strided copy behind that moves 0.4-1.9 TB/s at
// 1500 x 2000 x 192, the tiled transpose below is bound by HBM like any other streaming kernel.

#include "mp_common.h"

using namespace mpl;

namespace {

constexpr int kTile = 64;

// src (batch, rows, cols) -> dst (batch, cols, rows).  One 64 x 64 tile per workgroup of 64 x 4
// threads: rows of 256 contiguous bytes in, through LDS (padded against bank conflicts), rows of
// 256 contiguous bytes out.
__global__ void __launch_bounds__(256) transpose_kernel(const float* __restrict__ src,
                                                        float* __restrict__ dst, int64_t rows,
                                                        int64_t cols, int long_rows) {
  __shared__ float tile[kTile][kTile + 1];
  const int tx = threadIdx.x, ty = threadIdx.y;
  // the long side of the matrix runs along the grid's x axis
  const int64_t r0 = (int64_t)(long_rows ? blockIdx.x : blockIdx.y) * kTile;
  const int64_t c0 = (int64_t)(long_rows ? blockIdx.y : blockIdx.x) * kTile;
  const int64_t plane = rows * cols;
  const float* s = src + (int64_t)blockIdx.z * plane;
  float* d = dst + (int64_t)blockIdx.z * plane;
#pragma unroll
  for (int k = 0; k < kTile; k += 4) {
    const int64_t r = r0 + ty + k, c = c0 + tx;
    if (r < rows && c < cols) tile[ty + k][tx] = __builtin_nontemporal_load(s + r * cols + c);
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kTile; k += 4) {
    const int64_t c = c0 + ty + k, r = r0 + tx;
    if (r < rows && c < cols) __builtin_nontemporal_store(tile[tx][ty + k], d + c * rows + r);
  }
}

}  // namespace

extern "C" {

int mpl_transpose(const float* src, float* dst, int batch, int64_t rows, int64_t cols,
                  void* stream) {
  if (src == nullptr || dst == nullptr) return fail(MPL_EINVAL, "transpose: null pointer");
  if (batch < 0 || rows < 0 || cols < 0) return fail(MPL_EINVAL, "transpose: negative size");
  if (batch == 0 || rows == 0 || cols == 0) return MPL_OK;
  // the shorter side goes on the grid's y axis (65535 tiles at most)
  const int long_rows = rows > cols ? 1 : 0;
  const int64_t ny = ((long_rows ? cols : rows) + kTile - 1) / kTile;
  const int64_t nx = ((long_rows ? rows : cols) + kTile - 1) / kTile;
  if (ny > 65535 || nx > 0x7fffffff || batch > 65535)
    return fail(MPL_EINVAL, "transpose: too large (the shorter side must stay below 4 M elements)");
  const dim3 grid((unsigned)nx, (unsigned)ny, (unsigned)batch), block(kTile, 4);
  transpose_kernel<<<grid, block, 0, (hipStream_t)stream>>>(src, dst, rows, cols, long_rows);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MPL_ELAUNCH, "transpose: %s", hipGetErrorString(e));
  return MPL_OK;
}

}  // extern "C"
