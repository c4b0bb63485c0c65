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

#include <mutex>

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

// the body of both entry points; sums: 16 doubles of device scratch (kernel_cue_binary only)
int edge_shift_run(const char* who, int mode, const float* image, int batch, int channels,
                   int height, int width, int n_dirs, float sigma, float threshold, float penalty,
                   float* out, double* sums, hipStream_t st) {
  if (n_dirs == 0) return MPL_OK;
  const bool reduce = mode == MPL_EDGE_SUPERPIXEL || mode == MPL_EDGE_CUE_REAL ||
                      mode == MPL_EDGE_CUE_BINARY || mode == MPL_EDGE_THRESHOLD;
  const int64_t HW = (int64_t)height * width;
  if (!reduce) {
    edge_shift_channel_kernel<<<blocks_for((int64_t)batch * channels * HW), 256, 0, st>>>(
        image, mode, n_dirs, batch, channels, height, width, out);
  } else {
    if (mode != MPL_EDGE_CUE_BINARY) sums = nullptr;
    // cleared by a kernel, not a memset node: the call may be captured into a graph
    if (sums != nullptr) zero_sums_kernel<<<1, kWave, 0, st>>>(sums, kMaxDirs);
    edge_shift_reduce_kernel<<<blocks_for(HW), 256, 0, st>>>(image, mode, n_dirs, channels, height,
                                                            width, sigma, threshold, penalty, out,
                                                            sums);
    if (sums != nullptr)
      edge_binarize_kernel<<<blocks_for((int64_t)channels * HW), 256, 0, st>>>(
          n_dirs, channels, height, width, sums, out);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MPL_ELAUNCH, "%s: %s", who, hipGetErrorString(e));
  return MPL_OK;
}

int edge_shift_check(const char* who, int mode, const float* image, int batch, int channels,
                     int height, int width, int n_dirs, const float* out) {
  if (image == nullptr || out == nullptr) return fail(MPL_EINVAL, "%s: null tensor pointer", who);
  if (batch < 1 || channels < 1 || height < 1 || width < 1)
    return fail(MPL_EINVAL, "%s: batch/channels/height/width must be positive", who);
  if (n_dirs < 0 || n_dirs > kMaxDirs)
    return fail(MPL_EINVAL, "%s: n_dirs must be in [0, %d], got %d", who, kMaxDirs, n_dirs);
  if (mode < 0 || mode >= MPL_EDGE_MODES) return fail(MPL_EINVAL, "%s: unknown mode %d", who, mode);
  if ((int64_t)height * width > 0x7fffffff) return fail(MPL_EINVAL, "%s: more than 2^31 pixels", who);
  const bool reduce = mode == MPL_EDGE_SUPERPIXEL || mode == MPL_EDGE_CUE_REAL ||
                      mode == MPL_EDGE_CUE_BINARY || mode == MPL_EDGE_THRESHOLD;
  if (reduce && batch != 1)
    return fail(MPL_EINVAL, "%s: the channel-reducing modes take one image (batch == 1)", who);
  return MPL_OK;
}

// ------------------------------------------------------------------------------------------------
// Library-owned scratch of mpl_edge_shift_static: the per-direction sums of kernel_cue_binary, one
// double per direction of the 16-direction table (128 bytes).  Every GPU the library runs on holds
// its own copy of this array, at its own address, until the process ends.  In host code the name
// is only a handle for hipGetSymbolAddress: kernels and fills take the resolved device pointer.
// ------------------------------------------------------------------------------------------------
constexpr int kStaticSums = MPL_MAX_DIRS;  // the most directions one call can ask for
static __device__ __align__(256) double scratch[kStaticSums];

constexpr int kMaxDevices = 64;
double* g_scratch_ptr[kMaxDevices];  // resolved address of `scratch` per device, null until asked
std::mutex g_scratch_mu;

// address of this device's copy of `scratch`; resolved once per device, with that device current
int static_sums(const char* who, double** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MPL_ELAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(MPL_EINVAL, "%s: device ordinal %d outside [0, %d)", who, dev, kMaxDevices);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    double* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(MPL_ELAUNCH, "%s: hipGetSymbolAddress(scratch) on device %d: %s", who, dev,
                  hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MPL_OK;
}

}  // namespace

extern "C" {

int mpl_edge_shift(int mode, const float* image, int batch, int channels, int height, int width,
                   int n_dirs, float sigma, float threshold, float penalty, float* out,
                   double* dir_sums, void* stream) {
  int rc = edge_shift_check("edge_shift", mode, image, batch, channels, height, width, n_dirs, out);
  if (rc != MPL_OK) return rc;
  if (mode == MPL_EDGE_CUE_BINARY && dir_sums == nullptr)
    return fail(MPL_EINVAL, "edge_shift: kernel_cue_binary needs the dir_sums scratch (16 doubles)");
  return edge_shift_run("edge_shift", mode, image, batch, channels, height, width, n_dirs, sigma,
                        threshold, penalty, out, dir_sums, (hipStream_t)stream);
}

int mpl_edge_shift_static(int mode, const float* image, int batch, int channels, int height,
                          int width, int n_dirs, float sigma, float threshold, float penalty,
                          float* out, void* stream) {
  const char* who = "edge_shift_static";
  if (n_dirs > kStaticSums)
    return fail(MPL_EINVAL, "%s: %d directions asked for, the library's static scratch holds the "
                "sums of at most %d", who, n_dirs, kStaticSums);
  int rc = edge_shift_check(who, mode, image, batch, channels, height, width, n_dirs, out);
  if (rc != MPL_OK) return rc;
  double* sums = nullptr;
  if ((rc = static_sums(who, &sums)) != MPL_OK) return rc;
  // the array keeps the previous call's sums: edge_shift_run clears it before it accumulates
  return edge_shift_run(who, mode, image, batch, channels, height, width, n_dirs, sigma, threshold,
                        penalty, out, sums, (hipStream_t)stream);
}

}  // extern "C"
