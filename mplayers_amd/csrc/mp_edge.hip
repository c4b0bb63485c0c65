// Edge-weight producer for gfx950: per-direction "shift and compare" maps of an image, the input
// the message-passing layers take as edge_weights.  Follows getEdgeShift of the reference
// (utils/edge_weights.py:45-111): for direction d with step r_d (table of MPLayers/common.cpp:28-76)
// and every pixel p whose front neighbour q = p - r_d lies inside the image
//     diff = |I(p) - I(q)|        (per channel)
//     out[d, p] = f_mode(diff)    (0 where q is outside the image)
// The weight is stored at the receiving pixel p, which is where the scan kernels read it.
//
// One thread per pixel (per channel for the per-channel modes) computes all directions, so the centre
// value is read once; the image is small next to the n_dirs output planes, so the kernel is bound
// by its writes.

#include "mp_common.h"

using namespace mpl;

namespace {

// cue modes: mean over channels of diff^2
__device__ __forceinline__ float mean_sq_diff(const float* __restrict__ img, int64_t p, int64_t q,
                                              int C, int64_t HW) {
  float acc = 0.f;
  for (int c = 0; c < C; ++c) {
    const float d = fabsf(img[(int64_t)c * HW + p] - img[(int64_t)c * HW + q]);
    acc += d * d;
  }
  return acc / (float)C;
}

// Per-channel modes: one thread per (b, c, h, w).
__global__ void __launch_bounds__(256) edge_shift_channel_kernel(
    const float* __restrict__ img, int mode, int n_dirs, int B, int C, int H, int W,
    float* __restrict__ out) {
  const int64_t HW = (int64_t)H * W;
  const int64_t total = (int64_t)B * C * HW;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t plane = i / HW;
    const int pix = (int)(i - plane * HW);
    const int h = pix / W, w = pix - h * W;
    const float cur = img[i];
    for (int d = 0; d < n_dirs; ++d) {
      int hs, ws;
      dir_step(d, &hs, &ws);
      const int qh = h - hs, qw = w - ws;
      float v = 0.f;
      if (qh >= 0 && qh < H && qw >= 0 && qw < W) {
        const float front = img[plane * HW + (int64_t)qh * W + qw];
        float diff = fabsf(cur - front);
        switch (mode) {
          case MPL_EDGE_GT:  // ground-truth label map: 255 marks a void boundary
            if (cur == 255.f) diff = 1.f;
            v = (diff == 0.f) ? 1.f : 0.f;
            break;
          case MPL_EDGE_CANNY:  // binary edge map: an edge pixel (1) always cuts
            if (cur == 1.f) diff = 1.f;
            v = 1.f - diff;
            break;
          case MPL_EDGE_LINEAR:
            v = 1.f - diff;
            break;
          case MPL_EDGE_EXP:
            v = expf(-diff);
            break;
          default:  // MPL_EDGE_SHIFT: the front neighbour's value itself
            v = front;
            break;
        }
      }
      out[(int64_t)d * total + i] = v;
    }
  }
}

// Channel-reducing modes (batch of one): one thread per (h, w); the value is written to every
// channel plane of the output, as the reference's broadcasting assignment does.
// sums (may be null): per-direction sum of the values over the pixels that have a front neighbour.
__global__ void __launch_bounds__(256) edge_shift_reduce_kernel(
    const float* __restrict__ img, int mode, int n_dirs, int C, int H, int W, float sigma,
    float threshold, float penalty, float* __restrict__ out, double* __restrict__ sums) {
  const int64_t HW = (int64_t)H * W;
  const int64_t total = (int64_t)C * HW;
  __shared__ double part[MPL_MAX_DIRS];
  if (threadIdx.x < MPL_MAX_DIRS) part[threadIdx.x] = 0.0;
  __syncthreads();
  for (int64_t base = (int64_t)blockIdx.x * blockDim.x; base < HW;
       base += (int64_t)gridDim.x * blockDim.x) {
    const int64_t p = base + threadIdx.x;
    const bool in = p < HW;
    const int h = in ? (int)(p / W) : 0, w = in ? (int)(p - (int64_t)h * W) : 0;
    for (int d = 0; d < n_dirs; ++d) {
      int hs, ws;
      dir_step(d, &hs, &ws);
      const int qh = h - hs, qw = w - ws;
      const bool has_front = in && qh >= 0 && qh < H && qw >= 0 && qw < W;
      float v = 0.f;
      if (has_front) {
        const int64_t q = (int64_t)qh * W + qw;
        if (mode == MPL_EDGE_SUPERPIXEL) {
          float s = 0.f;
          for (int c = 0; c < C; ++c) s += fabsf(img[(int64_t)c * HW + p] - img[(int64_t)c * HW + q]);
          v = (s == 0.f) ? 1.f : 0.f;
        } else {
          const float m = mean_sq_diff(img, p, q, C, HW);
          if (mode == MPL_EDGE_THRESHOLD)
            v = (m < threshold) ? penalty : 0.f;
          else
            v = expf(m / (-2.f * sigma * sigma));
        }
      }
      if (in) {
        for (int c = 0; c < C; ++c) out[(int64_t)d * total + (int64_t)c * HW + p] = v;
      }
      if (sums != nullptr) {
        const float ws_sum = wave_sum(has_front ? v : 0.f);
        if ((threadIdx.x & (kWave - 1)) == 0) atomicAdd(&part[d], (double)ws_sum);
      }
    }
  }
  if (sums != nullptr) {
    __syncthreads();
    if (threadIdx.x < n_dirs) atomicAdd(&sums[threadIdx.x], part[threadIdx.x]);
  }
}

// kernel_cue_binary: out = (value >= 0.8 * mean over the pixels that have a front neighbour)
__global__ void __launch_bounds__(256) edge_binarize_kernel(int n_dirs, int C, int H, int W,
                                                            const double* __restrict__ sums,
                                                            float* __restrict__ out) {
  const int64_t HW = (int64_t)H * W;
  const int64_t total = (int64_t)C * HW;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int pix = (int)(i % HW);
    const int h = pix / W, w = pix - h * W;
    for (int d = 0; d < n_dirs; ++d) {
      int hs, ws;
      dir_step(d, &hs, &ws);
      const int qh = h - hs, qw = w - ws;
      if (qh < 0 || qh >= H || qw < 0 || qw >= W) continue;  // stays 0
      const int ah = hs < 0 ? -hs : hs, aw = ws < 0 ? -ws : ws;
      const double count = (double)(H - ah) * (double)(W - aw);
      const float mean = (float)(sums[d] / count);
      const int64_t o = (int64_t)d * total + i;
      out[o] = (out[o] >= 0.8f * mean) ? 1.f : 0.f;
    }
  }
}

__global__ void zero_sums_kernel(double* sums, int n) {
  if ((int)threadIdx.x < n) sums[threadIdx.x] = 0.0;
}

int blocks_for(int64_t n) {
  int64_t b = (n + 255) / 256;
  if (b < 1) b = 1;
  if (b > 256 * 32) b = 256 * 32;
  return (int)b;
}

int edge_fail(const char* msg) { return fail(MPL_EINVAL, "%s", msg); }

}  // namespace

extern "C" {

int mpl_edge_shift(int mode, const float* image, int batch, int channels, int height, int width,
                   int n_dirs, float sigma, float threshold, float penalty, float* out,
                   double* dir_sums, void* stream) {
  if (image == nullptr || out == nullptr) return edge_fail("edge_shift: null tensor pointer");
  if (batch < 1 || channels < 1 || height < 1 || width < 1)
    return edge_fail("edge_shift: batch/channels/height/width must be positive");
  if (n_dirs < 0 || n_dirs > kMaxDirs) return edge_fail("edge_shift: n_dirs must be in [0, 16]");
  if (mode < 0 || mode >= MPL_EDGE_MODES) return edge_fail("edge_shift: unknown mode");
  if ((int64_t)height * width > 0x7fffffff) return edge_fail("edge_shift: more than 2^31 pixels");
  const bool reduce = mode == MPL_EDGE_SUPERPIXEL || mode == MPL_EDGE_CUE_REAL ||
                      mode == MPL_EDGE_CUE_BINARY || mode == MPL_EDGE_THRESHOLD;
  if (reduce && batch != 1)
    return edge_fail("edge_shift: the channel-reducing modes take one image (batch == 1)");
  if (mode == MPL_EDGE_CUE_BINARY && dir_sums == nullptr)
    return edge_fail("edge_shift: kernel_cue_binary needs the dir_sums scratch (16 doubles)");
  if (n_dirs == 0) return MPL_OK;
  hipStream_t st = (hipStream_t)stream;
  const int64_t HW = (int64_t)height * width;
  if (!reduce) {
    edge_shift_channel_kernel<<<blocks_for((int64_t)batch * channels * HW), 256, 0, st>>>(
        image, mode, n_dirs, batch, channels, height, width, out);
  } else {
    double* sums = (mode == MPL_EDGE_CUE_BINARY) ? dir_sums : nullptr;
    if (sums != nullptr) zero_sums_kernel<<<1, kWave, 0, st>>>(sums, kMaxDirs);
    edge_shift_reduce_kernel<<<blocks_for(HW), 256, 0, st>>>(image, mode, n_dirs, channels, height,
                                                            width, sigma, threshold, penalty, out,
                                                            sums);
    if (sums != nullptr)
      edge_binarize_kernel<<<blocks_for((int64_t)channels * HW), 256, 0, st>>>(
          n_dirs, channels, height, width, sums, out);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MPL_ELAUNCH, "edge_shift: %s", hipGetErrorString(e));
  return MPL_OK;
}

}  // extern "C"
