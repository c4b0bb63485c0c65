// MRF terms either side of the message-passing layers, for gfx950.
//
// Upstream: the stereo data term ("disparity space image") and the gradient cues that the reference
// computes on the host from an image pair (MPLayers/aux/aux.cpp:5-98 computeDSI, :100-170
// computeCues, called from MPLayers/aux/auxPy.cpp:62-103).  The cost volume comes out as (H, W, L)
// fp32, label axis innermost, which is the layout the layers take as `unary`.
//
// Downstream: the energy of a labelling, E = sum_p unary[p, x_p] + sum_(p,q) w_pq * ctx(x_p, x_q),
// which the reference evaluates off-line for its energy curves (tools/matlab/MRF/calEnergy.m:2-48)
// from the per-iteration labellings the layers save.
//
// All of it is integer or gather work bound by HBM writes (the cost volume) or by launch latency
// (everything else); the arithmetic of the data term is integer and therefore bit-exact.

#include "mp_common.h"

using namespace mpl;

namespace {

struct DsiParams {
  const uint8_t* im1;
  const uint8_t* im2;
  float* dsi;
  int H, W, bands, colors, L;
  int birchfield, squared, max_sum, bad_cost;
};

// Birchfield-Tomasi sampling-insensitive difference of one colour band (aux.cpp:56-70): the
// intensity of each image is compared with the range the other one spans between its half-way
// interpolants to the left and to the right.  All quantities are non-negative integers, `/ 2`
// truncates.
__device__ __forceinline__ int bt_diff(const uint8_t* p1, const uint8_t* p2, int bands, bool first1,
                                       bool last1, bool first2, bool last2) {
  const int c1 = p1[0];
  const int l1 = first1 ? c1 : (c1 + p1[-bands]) / 2;
  const int r1 = last1 ? c1 : (c1 + p1[bands]) / 2;
  const int c2 = p2[0];
  const int l2 = first2 ? c2 : (c2 + p2[-bands]) / 2;
  const int r2 = last2 ? c2 : (c2 + p2[bands]) / 2;
  const int min1 = min(c1, min(l1, r1)), max1 = max(c1, max(l1, r1));
  const int min2 = min(c2, min(l2, r2)), max2 = max(c2, max(l2, r2));
  const int d1 = max(0, max(c1 - max2, min2 - c1));
  const int d2 = max(0, max(c2 - max1, min1 - c2));
  return min(d1, d2);
}

__device__ __forceinline__ float dsi_value(const DsiParams& P, int y, int x, int d) {
  const int x2 = x - d;
  if (x2 < 0) return (float)P.bad_cost;
  const uint8_t* p1 = P.im1 + ((int64_t)y * P.W + x) * P.bands;
  const uint8_t* p2 = P.im2 + ((int64_t)y * P.W + x2) * P.bands;
  int sum = 0;
  for (int b = 0; b < P.colors; ++b) {
    int diff;
    if (P.birchfield) {
      diff = bt_diff(p1 + b, p2 + b, P.bands, x == 0, x == P.W - 1, x2 == 0, x2 == P.W - 1);
    } else {
      diff = abs((int)p1[b] - (int)p2[b]);
    }
    sum += P.squared ? diff * diff : diff;
  }
  return (float)min(sum, P.max_sum);
}

// Four consecutive disparities d0..d0+3 of one pixel.  The right image is read once for the six
// pixels x-d0+1 .. x-d0-4 that the four matches and their neighbours cover; a neighbour index
// clamped to the row makes the half-way interpolant at a row end equal the pixel itself, which is
// what the reference's special cases do.
__device__ __forceinline__ void dsi_quad(const DsiParams& P, int y, int x, int d0, float v[4]) {
  const uint8_t* row1 = P.im1 + (int64_t)y * P.W * P.bands;
  const uint8_t* row2 = P.im2 + (int64_t)y * P.W * P.bands;
  const int last = P.W - 1;
  const int xl = max(x - 1, 0) * P.bands, xc = x * P.bands, xr = min(x + 1, last) * P.bands;
  int pos[6];
#pragma unroll
  for (int j = 0; j < 6; ++j) pos[j] = min(max(x - d0 + 1 - j, 0), last) * P.bands;
  int sum[4] = {0, 0, 0, 0};
  for (int b = 0; b < P.colors; ++b) {
    const int c1 = row1[xc + b];
    int t[6];
#pragma unroll
    for (int j = 0; j < 6; ++j) t[j] = row2[pos[j] + b];
    if (P.birchfield) {
      const int l1 = (c1 + (int)row1[xl + b]) >> 1, r1 = (c1 + (int)row1[xr + b]) >> 1;
      const int lo1 = min(c1, min(l1, r1)), hi1 = max(c1, max(l1, r1));
      int half[5];
#pragma unroll
      for (int j = 0; j < 5; ++j) half[j] = (t[j] + t[j + 1]) >> 1;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int c2 = t[k + 1];
        const int lo2 = min(c2, min(half[k], half[k + 1]));
        const int hi2 = max(c2, max(half[k], half[k + 1]));
        const int d1 = max(0, max(c1 - hi2, lo2 - c1));
        const int d2 = max(0, max(c2 - hi1, lo1 - c2));
        const int diff = min(d1, d2);
        sum[k] += P.squared ? diff * diff : diff;
      }
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int diff = abs(c1 - t[k + 1]);
        sum[k] += P.squared ? diff * diff : diff;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k)
    v[k] = (float)(x - d0 - k < 0 ? P.bad_cost : min(sum[k], P.max_sum));
}

// One thread per 4 consecutive floats of the (H, W, L) volume: 16-byte stores, whatever L is.  The
// block's first element is decoded with wave-uniform 64-bit arithmetic, the thread's own offset
// from there with 32-bit divisions.
__global__ void __launch_bounds__(256) dsi_kernel(DsiParams P, int64_t total) {
  const int64_t base = (int64_t)blockIdx.x * 1024;
  const int64_t e0 = base + 4 * (int)threadIdx.x;
  if (e0 >= total) return;
  const int64_t pix_base = base / P.L;
  const unsigned r = (unsigned)(base - pix_base * P.L) + 4u * threadIdx.x;
  const unsigned pix_off = r / (unsigned)P.L;
  int d = (int)(r - pix_off * (unsigned)P.L);
  const int64_t y_base = pix_base / P.W;
  const unsigned xr = (unsigned)(pix_base - y_base * P.W) + pix_off;
  const unsigned y_off = xr / (unsigned)P.W;
  int x = (int)(xr - y_off * (unsigned)P.W);
  int y = (int)y_base + (int)y_off;
  float v[4];
  const int n = (int)min((int64_t)4, total - e0);
  if (d + 3 < P.L) {  // n == 4 follows: the pixel's labels end inside the volume
    dsi_quad(P, y, x, d, v);
  } else {
    for (int k = 0; k < 4; ++k) {
      v[k] = 0.f;
      if (k < n) {
        v[k] = dsi_value(P, y, x, d);
        if (++d == P.L) {
          d = 0;
          if (++x == P.W) {
            x = 0;
            ++y;
          }
        }
      }
    }
  }
  if (n == 4) {
    *reinterpret_cast<float4*>(P.dsi + e0) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    for (int k = 0; k < n; ++k) P.dsi[e0 + k] = v[k];
  }
}

// Gradient cues (aux.cpp:100-170): penalty where the squared colour difference to the right / lower
// neighbour is below nColors * thresh^2, else 1.  h_cue is (H, W-1) row-major, v_cue is (W, H-1)
// (column-major over the image), as auxPy.cpp:88-96 lays them out.
__global__ void __launch_bounds__(256) cues_kernel(const uint8_t* __restrict__ im, int H, int W,
                                                   int bands, int colors, int thresh_sq,
                                                   float penalty, float* __restrict__ h_cue,
                                                   float* __restrict__ v_cue) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)H * W) return;
  const int y = (int)(i / W), x = (int)(i - (int64_t)y * W);
  const uint8_t* p = im + i * bands;
  if (x < W - 1) {
    int s = 0;
    for (int b = 0; b < colors; ++b) {
      const int dx = (int)p[b] - (int)p[bands + b];
      s += dx * dx;
    }
    h_cue[(int64_t)y * (W - 1) + x] = s < thresh_sq ? penalty : 1.f;
  }
  if (y < H - 1) {
    int s = 0;
    for (int b = 0; b < colors; ++b) {
      const int dy = (int)p[b] - (int)p[(int64_t)W * bands + b];
      s += dy * dy;
    }
    v_cue[(int64_t)x * (H - 1) + y] = s < thresh_sq ? penalty : 1.f;
  }
}

__global__ void zero_doubles_kernel(double* out, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) out[i] = 0.0;
}

struct EnergyParams {
  const float* unary;      // (B, H, W, L)
  const float* context;    // L floats (1-D) or L x L (2-D, upper triangle read)
  const float* edge;       // (n_dir, B, H, W) or null (all weights 1)
  const uint8_t* labels;   // (n_lab, B, H, W)
  double* out;             // (n_lab, 2): unary energy, pairwise energy
  int n_dir, B, H, W, L, ctx2d;
};

__device__ __forceinline__ double block_sum(double v, double* lds) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) lds[wave] = v;
  __syncthreads();
  double total = 0.0;
  if (threadIdx.x == 0)
    for (int w = 0; w < (int)(blockDim.x >> 6); ++w) total += lds[w];
  __syncthreads();
  return total;  // valid in thread 0
}

// One thread per pixel of one labelling (blockIdx.y).  Every undirected edge is counted once,
// through the even direction of its pair: the edge between p and q = p - r_d carries the weight
// stored at the receiving pixel p, as in the scans.
__global__ void __launch_bounds__(256) energy_kernel(EnergyParams P) {
  __shared__ double lds[8];
  const int64_t HW = (int64_t)P.H * P.W, BHW = HW * P.B;
  const uint8_t* lab = P.labels + (int64_t)blockIdx.y * BHW;
  double eu = 0.0, ep = 0.0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < BHW;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t b = i / HW;
    const int pix = (int)(i - b * HW);
    const int h = pix / P.W, w = pix - h * P.W;
    const int xp = lab[i];
    if (xp < P.L) eu += (double)P.unary[i * P.L + xp];
    for (int d = 0; d < P.n_dir; d += 2) {
      int hs, ws;
      dir_step(d, &hs, &ws);
      const int qh = h - hs, qw = w - ws;
      if (qh < 0 || qh >= P.H || qw < 0 || qw >= P.W) continue;
      const int xq = lab[b * HW + (int64_t)qh * P.W + qw];
      if (xp >= P.L || xq >= P.L) continue;
      const float c = P.ctx2d ? P.context[min(xp, xq) * P.L + max(xp, xq)]
                              : P.context[abs(xp - xq)];
      const float wt = P.edge ? P.edge[(int64_t)d * BHW + i] : 1.f;
      ep += (double)wt * (double)c;
    }
  }
  eu = block_sum(eu, lds);
  ep = block_sum(ep, lds);
  if (threadIdx.x == 0) {
    atomicAdd(P.out + 2 * blockIdx.y, eu);
    atomicAdd(P.out + 2 * blockIdx.y + 1, ep);
  }
}

int terms_fail(const char* msg) { return fail(MPL_EINVAL, "%s", msg); }

int launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MPL_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return MPL_OK;
}

}  // namespace

extern "C" {

int mpl_stereo_data_cost(const uint8_t* left, const uint8_t* right, int height, int width,
                         int bands, int n_labels, int birchfield, int squared_diffs,
                         int trunc_diffs, float* data_cost, void* stream) {
  if (left == nullptr || right == nullptr || data_cost == nullptr)
    return terms_fail("stereo_data_cost: null pointer");
  if (height < 1 || width < 1 || bands < 1 || n_labels < 1)
    return terms_fail("stereo_data_cost: height/width/bands/n_labels must be positive");
  if ((int64_t)height * width > 0x7fffffff)
    return terms_fail("stereo_data_cost: more than 2^31 pixels");
  DsiParams P;
  P.im1 = left;
  P.im2 = right;
  P.dsi = data_cost;
  P.H = height;
  P.W = width;
  P.bands = bands;
  P.colors = bands < 3 ? bands : 3;
  P.L = n_labels;
  P.birchfield = birchfield != 0;
  P.squared = squared_diffs != 0;
  // aux.cpp:24-31: the truncation is per colour for absolute differences, Euclidean for squared
  // ones; out-of-image matches cost the smaller of the worst match and the truncation.
  const int worst = P.colors * (P.squared ? 255 * 255 : 255);
  P.max_sum = P.squared ? trunc_diffs * trunc_diffs : P.colors * abs(trunc_diffs);
  P.bad_cost = worst < P.max_sum ? worst : P.max_sum;
  const int64_t total = (int64_t)height * width * n_labels;
  const int64_t blocks = (total + 1023) / 1024;
  if (blocks > 0x7fffffff) return terms_fail("stereo_data_cost: cost volume too large");
  dsi_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(P, total);
  return launch_status("stereo_data_cost");
}

int mpl_gradient_cues(const uint8_t* image, int height, int width, int bands, int grad_thresh,
                      float grad_penalty, float* h_cue, float* v_cue, void* stream) {
  if (image == nullptr) return terms_fail("gradient_cues: null image");
  if (height < 1 || width < 1 || bands < 1)
    return terms_fail("gradient_cues: height/width/bands must be positive");
  if ((h_cue == nullptr && width > 1) || (v_cue == nullptr && height > 1))
    return terms_fail("gradient_cues: null output");
  if ((int64_t)height * width > 0x7fffffff) return terms_fail("gradient_cues: more than 2^31 pixels");
  const int colors = bands < 3 ? bands : 3;
  const int64_t n = (int64_t)height * width;
  cues_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(
      image, height, width, bands, colors, grad_thresh * colors * grad_thresh, grad_penalty, h_cue,
      v_cue);
  return launch_status("gradient_cues");
}

int mpl_mrf_energy(const mpl_shape* shape, int n_labelings, const float* unary,
                   const float* context, const float* edge_weights, const uint8_t* labels,
                   double* energy, void* stream) {
  if (shape == nullptr || unary == nullptr || context == nullptr || labels == nullptr ||
      energy == nullptr)
    return terms_fail("mrf_energy: null pointer");
  if (shape->batch < 1 || shape->height < 1 || shape->width < 1 || shape->n_disp < 1 ||
      shape->n_disp > 256)
    return terms_fail("mrf_energy: batch/height/width must be positive, n_disp in [1, 256]");
  if (shape->n_dir < 0 || shape->n_dir > kMaxDirs || (shape->n_dir & 1))
    return terms_fail("mrf_energy: n_dir must be even and at most 16");
  if (n_labelings < 0 || n_labelings > 65535) return terms_fail("mrf_energy: n_labelings out of range");
  if ((int64_t)shape->height * shape->width > 0x7fffffff)
    return terms_fail("mrf_energy: more than 2^31 pixels");
  if (n_labelings == 0) return MPL_OK;
  hipStream_t st = (hipStream_t)stream;
  EnergyParams P;
  P.unary = unary;
  P.context = context;
  P.edge = edge_weights;
  P.labels = labels;
  P.out = energy;
  P.n_dir = shape->n_dir;
  P.B = shape->batch;
  P.H = shape->height;
  P.W = shape->width;
  P.L = shape->n_disp;
  P.ctx2d = shape->ctx2d;
  zero_doubles_kernel<<<1, 256, 0, st>>>(energy, 2 * n_labelings);
  const int64_t n = (int64_t)P.B * P.H * P.W;
  int64_t bx = (n + 255) / 256;
  if (bx > 4096) bx = 4096;
  energy_kernel<<<dim3((unsigned)bx, (unsigned)n_labelings), 256, 0, st>>>(P);
  return launch_status("mrf_energy");
}

}  // extern "C"
