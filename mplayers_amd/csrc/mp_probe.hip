// Bandwidth probes: what the memory system sustains for traffic of the scans' shape.
//
// The scan kernels are long-lived wavefronts, one per chain, that stream several planes in and out
// one pixel vector at a time.  These kernels move the same bytes in the same shape without any of
// the arithmetic (n_in planes read and summed, n_out planes written, register prefetch ring), and a
// one-pass streaming kernel moves them the way an element-wise kernel does, so the scans can be
// rated against what the hardware delivers for their access pattern rather than against the data
// sheet alone.  Diagnostics only; no counterpart in the reference.

#include "mp_common.h"

using namespace mpl;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kProbeDepth = 8;  // pixels in flight per wavefront, as in the scans

// One wavefront per chain; a pixel vector is `units` 16-byte pieces (lanes beyond that idle).
// Chain c starts at unit c * chain_stride, pixel t at + t * pix_stride.
template <int NIN, int NOUT>
__global__ void __launch_bounds__(kWave) chain_copy_kernel(const v4f* __restrict__ in,
                                                           v4f* __restrict__ out, int64_t plane,
                                                           int units, int64_t chain_stride,
                                                           int64_t pix_stride, int n_pix) {
  if ((int)threadIdx.x >= units) return;
  const int64_t base = (int64_t)blockIdx.x * chain_stride + threadIdx.x;
  v4f ring[kProbeDepth][NIN];
  v4f total = 0.f;
#pragma unroll
  for (int d = 0; d < kProbeDepth; ++d)
#pragma unroll
    for (int k = 0; k < NIN; ++k)
      ring[d][k] = __builtin_nontemporal_load(in + k * plane + base + (d < n_pix ? d : 0) * pix_stride);
  for (int t = 0; t < n_pix; t += kProbeDepth) {
#pragma unroll
    for (int d = 0; d < kProbeDepth; ++d) {
      v4f acc = ring[d][0];
#pragma unroll
      for (int k = 1; k < NIN; ++k) acc += ring[d][k];
      const int next = t + d + kProbeDepth;
      if (next < n_pix) {
#pragma unroll
        for (int k = 0; k < NIN; ++k)
          ring[d][k] = __builtin_nontemporal_load(in + k * plane + base + next * pix_stride);
      }
      if (t + d < n_pix) {
#pragma unroll
        for (int k = 0; k < NOUT; ++k)
          __builtin_nontemporal_store(acc + (float)k, out + k * plane + base + (t + d) * pix_stride);
        if (NOUT == 0) total += acc;
      }
    }
  }
  if (NOUT == 0 && total.x == 1.2345e30f) out[base] = total;  // keeps the loads alive
}

// One thread per 16 bytes, one pass, as the element-wise kernels.
template <int NIN, int NOUT>
__global__ void __launch_bounds__(256) stream_copy_kernel(const v4f* __restrict__ in,
                                                          v4f* __restrict__ out, int64_t plane) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= plane) return;
  v4f acc = __builtin_nontemporal_load(in + i);
#pragma unroll
  for (int k = 1; k < NIN; ++k) acc += __builtin_nontemporal_load(in + k * plane + i);
#pragma unroll
  for (int k = 0; k < NOUT; ++k) __builtin_nontemporal_store(acc + (float)k, out + k * plane + i);
  if (NOUT == 0 && acc.x == 1.2345e30f) out[i] = acc;
}

template <int NIN, int NOUT>
void launch_probe(int shape, const float* in, float* out, int H, int W, int L, hipStream_t st) {
  const int units = L / 4;
  const int64_t plane = (int64_t)H * W * units;
  const v4f* src = reinterpret_cast<const v4f*>(in);
  v4f* dst = reinterpret_cast<v4f*>(out);
  if (shape == MPL_PROBE_ROWS) {
    chain_copy_kernel<NIN, NOUT><<<H, kWave, 0, st>>>(src, dst, plane, units, (int64_t)W * units,
                                                      units, W);
  } else if (shape == MPL_PROBE_COLUMNS) {
    chain_copy_kernel<NIN, NOUT><<<W, kWave, 0, st>>>(src, dst, plane, units, units,
                                                      (int64_t)W * units, H);
  } else {
    stream_copy_kernel<NIN, NOUT><<<(unsigned)((plane + 255) / 256), 256, 0, st>>>(src, dst, plane);
  }
}

}  // namespace

extern "C" {

int mpl_probe_copy(int shape, int n_in, int n_out, const float* in, float* out, int height,
                   int width, int n_labels, void* stream) {
  if (in == nullptr || out == nullptr) return fail(MPL_EINVAL, "probe_copy: null pointer");
  if (shape < 0 || shape > MPL_PROBE_STREAM) return fail(MPL_EINVAL, "probe_copy: unknown shape");
  if (height < 1 || width < 1 || n_labels < 4 || n_labels > 256 || (n_labels & 3))
    return fail(MPL_EINVAL, "probe_copy: n_labels must be a multiple of 4 in [4, 256]");
  if ((int64_t)height * width * n_labels / 4 / 256 > 0x7fffffff)
    return fail(MPL_EINVAL, "probe_copy: plane too large");
  hipStream_t st = (hipStream_t)stream;
  const int key = n_in * 10 + n_out;
  switch (key) {
    case 11: launch_probe<1, 1>(shape, in, out, height, width, n_labels, st); break;
    case 13: launch_probe<1, 3>(shape, in, out, height, width, n_labels, st); break;
    case 30: launch_probe<3, 0>(shape, in, out, height, width, n_labels, st); break;
    case 32: launch_probe<3, 2>(shape, in, out, height, width, n_labels, st); break;
    case 43: launch_probe<4, 3>(shape, in, out, height, width, n_labels, st); break;
    default:
      return fail(MPL_EINVAL, "probe_copy: (n_in, n_out) must be one of (1,1) (1,3) (3,0) (3,2) (4,3)");
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MPL_ELAUNCH, "probe_copy: %s", hipGetErrorString(e));
  return MPL_OK;
}

}  // extern "C"
