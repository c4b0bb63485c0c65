// C ABI, host orchestration and the element-wise kernels of the TRWP / ISGMR path (gfx950).
// The scan kernels live in mp_fwd.hip / mp_bwd.hip; shared device helpers in mp_common.h.
//
// Traffic model: instead of re-summing all messages for every sweep (UpdateUnaryKernel of the
// reference, TRWP_forward.cu:60-80), a belief plane S = unary + sum_k m_k is kept, so a sweep of
// direction d reads S, m_d, m_inv and writes m_d (and S for TRWP): 20 B per label.  The backward
// pass keeps the gradient planes as g_k = A + h_k with one shared plane A (which ends up being
// dunary) for the same reason.

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "mp_common.h"

using namespace mpl;

namespace {

// 1-D context c[0..L-1]: find the constant tail and recognise a truncated linear table.  One wave,
// every lane looks at the entries lane, lane + 64, ...; the findings are combined with ballots.
__global__ void __launch_bounds__(kWave) analyze_context_kernel(const float* __restrict__ ctx, int L,
                                                                int ctx2d, CtxDesc* __restrict__ d) {
  const int lane = threadIdx.x;
  CtxDesc r;
  r.band_k = 0;
  r.c0_is_min = 0;
  r.cmax = 0.f;
  r.msg_nonzero = 0;
  r.linear = 0;
  r.slope = 0.f;
  if (!ctx2d) {
    const float tail = ctx[L - 1];
    const float c0 = ctx[0];
    const float slope = L >= 2 ? ctx[1] : 0.f;
    int last_ne = -1;  // largest index whose entry differs from the tail
    bool below = true, c0min = true, lin = true;
    for (int i = lane; i < L; i += kWave) {
      const float v = ctx[i];
      if (!(v == tail)) last_ne = i;
      below = below && (v <= tail);
      c0min = c0min && (c0 <= v);
      lin = lin && (v == fminf(slope * (float)i, tail));
    }
    int k = (int)-wave_min(-(float)last_ne) + 1;  // c[k..L-1] == tail  (indices < 2^24: exact)
    // a NaN tail disables both fast paths; tested on the bit pattern because the library is
    // compiled without NaN semantics, where `tail == tail` may be folded to true
    const bool tail_is_nan = (__builtin_bit_cast(unsigned, tail) & 0x7fffffffu) > 0x7f800000u;
    const bool ok = !tail_is_nan && ballot(!below) == 0;
    const bool all_c0min = ballot(!c0min) == 0;
    const bool all_lin = ballot(!lin) == 0;
    if (k < 1) k = 1;  // a constant context: the centre tap alone is the band
    if (ok && k <= kMaxBandK) {
      r.band_k = k;
      r.cmax = tail;
      r.c0_is_min = all_c0min ? 1 : 0;
    }
    // truncated linear, bit for bit: c[k] == min(c[1] * k, c[L-1])
    if (ok && L >= 2 && c0 == 0.f && slope >= 0.f && all_lin) {
      r.linear = 1;
      r.slope = slope;
      r.cmax = tail;
    }
  }
  if (lane == 0) *d = r;
}

// ------------------------------------------------------------------------------------------------
// elementwise kernels.  V floats per lane and access (4 when every plane is 16-byte aligned and the
// plane size is a multiple of 4, else 1); ND: number of directions when it is one of the usual ones
// (loads of all planes are then issued back to back), 0: run-time loop.
// ------------------------------------------------------------------------------------------------
#ifndef MPL_EW_NT
#define MPL_EW_NT 1  // planes are streamed once: non-temporal loads and stores
#endif
template <int V>
struct Pack {
  float v[V];
};
template <int V>
__device__ __forceinline__ Pack<V> ld_pack(const float* p) {
  Pack<V> r;
  if constexpr (V == 4) {
    const f32x4 t = MPL_EW_NT ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p))
                              : *reinterpret_cast<const f32x4*>(p);
    r.v[0] = t.x;
    r.v[1] = t.y;
    r.v[2] = t.z;
    r.v[3] = t.w;
  } else {
    r.v[0] = MPL_EW_NT ? __builtin_nontemporal_load(p) : *p;
  }
  return r;
}
template <int V>
__device__ __forceinline__ void st_pack(float* p, const Pack<V>& r) {
  if constexpr (V == 4) {
    f32x4 t;
    t.x = r.v[0];
    t.y = r.v[1];
    t.z = r.v[2];
    t.w = r.v[3];
    if (MPL_EW_NT)
      __builtin_nontemporal_store(t, reinterpret_cast<f32x4*>(p));
    else
      *reinterpret_cast<f32x4*>(p) = t;
  } else {
    if (MPL_EW_NT)
      __builtin_nontemporal_store(r.v[0], p);
    else
      *p = r.v[0];
  }
}

// S = unary + sum_k m_k  (k ascending, as UpdateUnaryKernel sums, TRWP_forward.cu:70-73)
template <int V, int ND>
__global__ void __launch_bounds__(256) belief_kernel(const float* __restrict__ unary,
                                                     const float* __restrict__ msg, int n_dir_rt,
                                                     int64_t N, float* __restrict__ S,
                                                     int* nonzero_flag, const int* only_if = nullptr) {
  // (only_if: a flag an earlier kernel of the stream has set or left clear; clear: nothing to do)
  if (only_if != nullptr && *only_if == 0) return;
  const int n_dir = ND > 0 ? ND : n_dir_rt;
  bool any = false;  // some message of this thread's elements is not zero
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V; i < N;
       i += (int64_t)gridDim.x * blockDim.x * V) {
    Pack<V> v = ld_pack<V>(unary + i);
    if constexpr (ND > 0) {
      Pack<V> m[ND];
#pragma unroll
      for (int k = 0; k < ND; ++k) m[k] = ld_pack<V>(msg + (int64_t)k * N + i);
#pragma unroll
      for (int k = 0; k < ND; ++k)
#pragma unroll
        for (int j = 0; j < V; ++j) {
          v.v[j] += m[k].v[j];
          any = any || (m[k].v[j] != 0.f);
        }
    } else {
      for (int k = 0; k < n_dir; ++k) {
        const Pack<V> m = ld_pack<V>(msg + (int64_t)k * N + i);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          v.v[j] += m.v[j];
          any = any || (m.v[j] != 0.f);
        }
      }
    }
    st_pack<V>(S + i, v);
  }
  if (nonzero_flag != nullptr && any) *nonzero_flag = 1;  // every writer stores the same value
}

// Sets *flag when some element of the n_dir message planes is not zero (every writer stores the
// same value).  The reference's callers pass cleared message tensors; knowing that on the device
// lets the first sweeps read the unary terms in place of planes that would have to be built first.
template <int V, int ND>
__global__ void __launch_bounds__(256) check_nonzero_kernel(const float* __restrict__ msg,
                                                            int n_dir_rt, int64_t N, int* flag) {
  const int n_dir = ND > 0 ? ND : n_dir_rt;
  bool any = false;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V; i < N;
       i += (int64_t)gridDim.x * blockDim.x * V) {
    if constexpr (ND > 0) {
      Pack<V> m[ND];
#pragma unroll
      for (int k = 0; k < ND; ++k) m[k] = ld_pack<V>(msg + (int64_t)k * N + i);
#pragma unroll
      for (int k = 0; k < ND; ++k)
#pragma unroll
        for (int j = 0; j < V; ++j) any = any || (m[k].v[j] != 0.f);
    } else {
      for (int k = 0; k < n_dir; ++k) {
        const Pack<V> m = ld_pack<V>(msg + (int64_t)k * N + i);
#pragma unroll
        for (int j = 0; j < V; ++j) any = any || (m.v[j] != 0.f);
      }
    }
  }
  if (any) *flag = 1;
}

// ISGMR: every direction of an iteration reads the old messages only through
//   U_d = rho * (unary + sum_k m_k - m_d) - m_{d^1}      (UpdateUnaryKernel, ISGMR_forward.cu:101-121)
// so U_d is stored once per iteration (in place of m_d, or into the other message buffer) before
// the sweeps: a sweep then reads one plane per pixel, not three.
template <int V, int ND>
__global__ void __launch_bounds__(256) isgmr_unary_kernel(const float* __restrict__ unary,
                                                          const float* msg, float* out,
                                                          int n_dir_rt, int64_t N, float rho,
                                                          int pair_share, const int* only_if = nullptr) {
  if (only_if != nullptr && *only_if == 0) return;  // (see belief_kernel)
  constexpr int KD = ND > 0 ? ND : kMaxDirs;
  const int n_dir = ND > 0 ? ND : n_dir_rt;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V; i < N;
       i += (int64_t)gridDim.x * blockDim.x * V) {
    Pack<V> S = ld_pack<V>(unary + i);
    Pack<V> m[KD];
#pragma unroll
    for (int k = 0; k < KD; ++k) {
      if (k < n_dir) {
        m[k] = ld_pack<V>(msg + (int64_t)k * N + i);
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) m[k].v[j] = 0.f;
      }
    }
#pragma unroll
    for (int k = 0; k < KD; ++k)
      if (k < n_dir) {
#pragma unroll
        for (int j = 0; j < V; ++j) S.v[j] += m[k].v[j];  // k ascending, as the reference sums
      }
#pragma unroll
    for (int k = 0; k < KD; ++k) {
      // pair_share (rho == 1): U_d and U_{d^1} are both S - m_d - m_{d^1}; one plane per pair is
      // stored (they differ by the order of the two subtractions, at most 2 ulp of S)
      if (k < n_dir && !(pair_share && (k & 1))) {
        Pack<V> u;
#pragma unroll
        for (int j = 0; j < V; ++j) u.v[j] = fmaf(S.v[j] - m[k].v[j], rho, -m[k ^ 1].v[j]);
        st_pack<V>(out + (int64_t)k * N + i, u);  // out == msg: in place
      }
    }
  }
}

// cost = factor*unary + sum_k m_k  (or + min_k m_k): CostAggregateKernel, TRWP_forward.cu:31-58,
// ISGMR_forward.cu:69-99.
template <int V, int ND>
__global__ void __launch_bounds__(256) aggregate_kernel(const float* __restrict__ unary,
                                                        const float* __restrict__ msg, int n_dir_rt,
                                                        int64_t N, float factor, int min_a_dir,
                                                        float* __restrict__ cost) {
  const int n_dir = ND > 0 ? ND : n_dir_rt;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V; i < N;
       i += (int64_t)gridDim.x * blockDim.x * V) {
    Pack<V> v = ld_pack<V>(unary + i);
#pragma unroll
    for (int j = 0; j < V; ++j) v.v[j] *= factor;
    Pack<V> mn;  // min_a_dir only
    auto fold = [&](int k, const Pack<V>& m) {
#pragma unroll
      for (int j = 0; j < V; ++j) {
        if (!min_a_dir)
          v.v[j] += m.v[j];  // ((unary + m_0) + m_1) + ... as the reference adds
        else if (k == 0)
          mn.v[j] = m.v[j];
        else
          mn.v[j] = (m.v[j] < mn.v[j]) ? m.v[j] : mn.v[j];
      }
    };
    if constexpr (ND > 0) {
      Pack<V> m[ND];
#pragma unroll
      for (int k = 0; k < ND; ++k) m[k] = ld_pack<V>(msg + (int64_t)k * N + i);
#pragma unroll
      for (int k = 0; k < ND; ++k) fold(k, m[k]);
    } else {
      for (int k = 0; k < n_dir; ++k) fold(k, ld_pack<V>(msg + (int64_t)k * N + i));
    }
    if (min_a_dir) {
#pragma unroll
      for (int j = 0; j < V; ++j) v.v[j] += mn.v[j];
    }
    st_pack<V>(cost + i, v);
  }
}

// label = argmin_l cost(l), smallest label on ties: CalLabelKernel, TRWP_forward.cu:8-29, with the
// cost of CostAggregateKernel recomputed on the fly.  One wave per pixel.
__global__ void __launch_bounds__(256) label_kernel(const float* __restrict__ unary,
                                                    const float* __restrict__ msg, int n_dir,
                                                    int64_t P, int L, float factor, int min_a_dir,
                                                    uint8_t* __restrict__ label) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t N = P * L;
  const int64_t wave0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
  const int64_t n_waves = ((int64_t)gridDim.x * blockDim.x) / kWave;
  for (int64_t pix = wave0; pix < P; pix += n_waves) {
    float best = INFINITY;
    int arg = 0x7fffffff;
    for (int l = lane; l < L; l += kWave) {
      int64_t i = pix * L + l;
      float v = unary[i] * factor;
      if (min_a_dir) {
        float mn = msg[i];
        for (int k = 1; k < n_dir; ++k) {
          float m = msg[(int64_t)k * N + i];
          if (m < mn) mn = m;
        }
        v += mn;
      } else {
        for (int k = 0; k < n_dir; ++k) v += msg[(int64_t)k * N + i];
      }
      if (v < best) {
        best = v;
        arg = l;
      }
    }
    float gmin = wave_min(best);
    // smallest label among the lanes that hold the minimum; a lane's own arg is its smallest
    float cand = (best == gmin) ? (float)arg : INFINITY;
    float amin = wave_min(cand);
    if (lane == 0) label[pix] = (uint8_t)((amin < (float)L) ? (int)amin : 0);
  }
}

// The same for label counts that are a multiple of 4: a group of `group` lanes (a power of two
// >= L/4) per pixel, 16 bytes per lane and plane, 64/group pixels per wavefront; the argmin is a
// butterfly over the group on (value, label) pairs.
__global__ void __launch_bounds__(256) label_quad_kernel(const float* __restrict__ unary,
                                                         const float* __restrict__ msg, int n_dir,
                                                         int64_t P, int L, int group, float factor,
                                                         int min_a_dir, uint8_t* __restrict__ label) {
  const int64_t N = P * L;
  const int sub = threadIdx.x & (group - 1);
  const int64_t pix = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / group;
  float best = INFINITY;
  int arg = 0x7fffffff;
  if (pix < P && sub * 4 < L) {
    const int64_t i = pix * L + sub * 4;
    Pack<4> v = ld_pack<4>(unary + i);
#pragma unroll
    for (int j = 0; j < 4; ++j) v.v[j] *= factor;
    if (min_a_dir) {
      Pack<4> mn = ld_pack<4>(msg + i);
      for (int k = 1; k < n_dir; ++k) {
        Pack<4> m = ld_pack<4>(msg + (int64_t)k * N + i);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (m.v[j] < mn.v[j]) mn.v[j] = m.v[j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) v.v[j] += mn.v[j];
    } else {
      for (int k = 0; k < n_dir; ++k) {
        Pack<4> m = ld_pack<4>(msg + (int64_t)k * N + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) v.v[j] += m.v[j];
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (v.v[j] < best) {
        best = v.v[j];
        arg = sub * 4 + j;
      }
  }
  for (int o = 1; o < group; o <<= 1) {
    float ob = __shfl_xor(best, o);
    int oa = __shfl_xor(arg, o);
    if (ob < best || (ob == best && oa < arg)) {
      best = ob;
      arg = oa;
    }
  }
  if (pix < P && sub == 0) label[pix] = (uint8_t)((arg < L) ? arg : 0);
}

static void launch_labels(const float* unary, const float* msg, int n_dir, int64_t P, int L,
                          float factor, int min_a_dir, uint8_t* label, hipStream_t st) {
  const bool aligned = (((uintptr_t)unary | (uintptr_t)msg) & 15) == 0;
  if ((L & 3) == 0 && aligned) {
    int group = 1;
    while (group * 4 < L) group <<= 1;
    const int64_t blocks = (P * group + 255) / 256;
    label_quad_kernel<<<(unsigned)blocks, 256, 0, st>>>(unary, msg, n_dir, P, L, group, factor,
                                                        min_a_dir, label);
  } else {
    const int64_t waves = (P < 256 * 64) ? P : 256 * 64;
    label_kernel<<<(int)((waves + 3) / 4), 256, 0, st>>>(unary, msg, n_dir, P, L, factor, min_a_dir,
                                                         label);
  }
}

// ISGMR: after all directions of an iteration have been scanned back (X_k = dU_k):
//   dunary += rho * sum_k X_k ;  gu_k = rho * (sum - X_k) - X_{k^1}   (written to G)
// (UpdateUnaryKernelBack summed over directions + SumMsgKernel, ISGMR_backward.cu:39-60, 482-483)
template <int V, int ND>
__global__ void __launch_bounds__(256) isgmr_combine_kernel(const float* X, float* G, int n_dir_rt,
                                                            int64_t N, float rho,
                                                            const float* __restrict__ dcost,
                                                            float factor, int init_dunary,
                                                            int write_gu, int pair_share,
                                                            float* __restrict__ dunary) {
  constexpr int KD = ND > 0 ? ND : kMaxDirs;
  const int n_dir = ND > 0 ? ND : n_dir_rt;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V; i < N;
       i += (int64_t)gridDim.x * blockDim.x * V) {
    Pack<V> x[KD];
#pragma unroll
    for (int k = 0; k < KD; ++k) {
      if (k < n_dir) {
        x[k] = ld_pack<V>(X + (int64_t)k * N + i);
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) x[k].v[j] = 0.f;
      }
    }
    Pack<V> du = init_dunary ? ld_pack<V>(dcost + i) : ld_pack<V>(dunary + i);
    Pack<V> sum;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      sum.v[j] = 0.f;
#pragma unroll
      for (int k = KD - 1; k >= 0; --k)
        if (k < n_dir) sum.v[j] += x[k].v[j];
      if (init_dunary) du.v[j] *= factor;
      du.v[j] = fmaf(rho, sum.v[j], du.v[j]);
    }
    st_pack<V>(dunary + i, du);
    if (write_gu) {
#pragma unroll
      for (int k = 0; k < KD; ++k) {
        // pair_share (rho == 1): gu_k and gu_{k^1} are both sum - X_k - X_{k^1}; one plane per
        // pair is stored (G == X: in place, every plane)
        if (k < n_dir && !(pair_share && (k & 1))) {
          Pack<V> g;
#pragma unroll
          for (int j = 0; j < V; ++j) g.v[j] = fmaf(rho, sum.v[j] - x[k].v[j], -x[k ^ 1].v[j]);
          st_pack<V>(G + (int64_t)k * N + i, g);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
thread_local char g_err[512] = "";

// Optional per-kernel timing with HIP events on the launch stream (off unless mpl_profile_begin
// was called): lets a benchmark read each kernel's average duration without an external profiler.
struct ProfRec {
  int kind;
  int sweeps;  // direction sweeps the launch stands for (2 for a fused pair)
  hipEvent_t start, stop;
};
struct Profiler {
  std::atomic<bool> on{false};
  std::vector<ProfRec> recs;
  std::vector<hipEvent_t> pool;
  hipEvent_t get_event() {
    if (!pool.empty()) {
      hipEvent_t e = pool.back();
      pool.pop_back();
      return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
  }
};
Profiler g_prof;
std::mutex g_prof_mu;

struct Timed {
  hipStream_t st;
  hipEvent_t stop = nullptr;
  Timed(int kind, hipStream_t s, int sweeps = 1) : st(s) {
    if (!g_prof.on.load(std::memory_order_acquire)) return;
    std::lock_guard<std::mutex> lk(g_prof_mu);
    ProfRec r;
    r.kind = kind;
    r.sweeps = sweeps;
    r.start = g_prof.get_event();
    r.stop = g_prof.get_event();
    if (r.start == nullptr || r.stop == nullptr) return;
    (void)hipEventRecord(r.start, st);
    stop = r.stop;
    g_prof.recs.push_back(r);
  }
  ~Timed() {
    if (stop != nullptr) (void)hipEventRecord(stop, st);
  }
};

int check_shape(const mpl_shape* s, int n_iter) {
  if (s == nullptr) return fail(MPL_EINVAL, "shape is null");
  if (s->n_dir < 2 || s->n_dir > kMaxDirs || (s->n_dir & 1))
    return fail(MPL_EINVAL, "n_dir must be even and in [2, %d], got %d", kMaxDirs, s->n_dir);
  if (s->batch < 1 || s->height < 1 || s->width < 1)
    return fail(MPL_EINVAL, "batch/height/width must be positive, got %d/%d/%d", s->batch,
                s->height, s->width);
  if (s->n_disp < 1 || s->n_disp > kMaxL)
    return fail(MPL_EINVAL, "n_disp must be in [1, %d] (uint8 argmin indices), got %d", kMaxL,
                s->n_disp);
  if (s->ctx2d && s->n_disp > kMaxCtx2dL)
    return fail(MPL_EINVAL, "a 2-D context table needs n_disp <= %d, got %d", kMaxCtx2dL,
                s->n_disp);
  if (n_iter < 1) return fail(MPL_EINVAL, "n_iter must be positive, got %d", n_iter);
  int64_t P = (int64_t)s->batch * s->height * s->width;
  if (P > 0x7fffffff) return fail(MPL_EINVAL, "more than 2^31 pixels");
  // pixels are addressed with 32-bit byte offsets from the first pixel of their batch item
  if ((int64_t)s->height * s->width * s->n_disp * 4 > kMaxImageBytes)
    return fail(MPL_EINVAL, "one batch item (height*width*n_disp floats) must stay below 4 GiB");
  int64_t max_blocks = 0;
  for (int d = 0; d < s->n_dir; ++d)
    max_blocks += (int64_t)s->batch * make_dir(d, s->height, s->width).n_chains;
  if (max_blocks > 0x7fffffff) return fail(MPL_EINVAL, "more than 2^31 chains");
  return MPL_OK;
}

int launch_ok(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MPL_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return MPL_OK;
}

// Workgroups of an element-wise kernel over n accesses (of 4 floats or of 1): one access per thread.
// One pass over the data with as many workgroups as it takes measured 3-8 % faster than a
// grid-stride loop of 32 workgroups per CU on the 2.3 GB planes, and 2 / 4 / 8 accesses per thread
// measured 2 / 5 / 9 % slower than one (workgroups of 64, 128 and 512 threads: 4 to 5 % slower than
// 256); the cap only bounds the grid.
#ifndef MPL_EW_BLOCKS_PER_CU
#define MPL_EW_BLOCKS_PER_CU 4096
#endif
int elementwise_blocks(int64_t n) {
  int64_t b = (n + 256 - 1) / 256;
  if (b < 1) b = 1;
  if (b > 256 * MPL_EW_BLOCKS_PER_CU) b = 256 * MPL_EW_BLOCKS_PER_CU;
  return (int)b;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Picks the instantiation of an element-wise kernel: 4 floats per access when the planes allow it,
// the direction count as a compile-time constant when it is 4, 8 or 16.
#define MPL_EW_LAUNCH(KERNEL, VEC4, NDIR, N, ST, ...)                                            \
  do {                                                                                           \
    const int blocks_ = elementwise_blocks((VEC4) ? (N) / 4 : (N));                              \
    if (VEC4) {                                                                                  \
      switch (NDIR) {                                                                            \
        case 4: KERNEL<4, 4><<<blocks_, 256, 0, ST>>>(__VA_ARGS__); break;                       \
        case 8: KERNEL<4, 8><<<blocks_, 256, 0, ST>>>(__VA_ARGS__); break;                       \
        case 16: KERNEL<4, 16><<<blocks_, 256, 0, ST>>>(__VA_ARGS__); break;                     \
        default: KERNEL<4, 0><<<blocks_, 256, 0, ST>>>(__VA_ARGS__); break;                      \
      }                                                                                          \
    } else {                                                                                     \
      KERNEL<1, 0><<<blocks_, 256, 0, ST>>>(__VA_ARGS__);                                        \
    }                                                                                            \
  } while (0)

void fill_dirs(const mpl_shape* s, int first, int count, int* dirs, int* prefix, int* n_dirs) {
  *n_dirs = count;
  prefix[0] = 0;
  for (int i = 0; i < count; ++i) {
    dirs[i] = first + i;
    prefix[i + 1] = prefix[i] + s->batch * make_dir(first + i, s->height, s->width).n_chains;
  }
}

int labels_per_lane(int L) { return (L + kWave - 1) / kWave; }

// process defaults of the per-call choices (mpl_set_option); a call reads them once
std::atomic<int> g_packed_scans{1};  // MPL_OPT_PACKED_SCANS: 0 off, 1 by chain count, 2 always
std::atomic<int> g_fused_u{1};       // MPL_OPT_FUSED_U
std::atomic<int> g_belief_rebuild{MPL_BELIEF_REBUILD_DEFAULT};  // MPL_OPT_BELIEF_REBUILD
std::atomic<int> g_split_waves{0};   // MPL_OPT_DENSE_SPLIT_WAVES: 0 = by the model of choose_split

// what one call does, from its flags and the process defaults
struct CallOpts {
  int packed;   // 0 off, 1 by chain count, 2 always
  bool fused_u;
  bool fused_pairs;
  bool dense_table;
};

int read_flags(unsigned flags, const char* what, CallOpts* o) {
  if (flags & ~MPL_F_ALL) return fail(MPL_EINVAL, "%s: unknown flag bits 0x%x", what, flags & ~MPL_F_ALL);
  if ((flags & MPL_F_PACKED_OFF) && (flags & MPL_F_PACKED_ALWAYS))
    return fail(MPL_EINVAL, "%s: MPL_F_PACKED_OFF and MPL_F_PACKED_ALWAYS exclude each other", what);
  o->packed = (flags & MPL_F_PACKED_OFF) ? 0
              : (flags & MPL_F_PACKED_ALWAYS) ? 2 : g_packed_scans.load(std::memory_order_relaxed);
  o->fused_u = (flags & MPL_F_FUSED_U_OFF) ? false : g_fused_u.load(std::memory_order_relaxed) != 0;
  o->fused_pairs = (flags & MPL_F_FUSED_PAIRS_OFF) == 0;
  o->dense_table = (flags & MPL_F_DENSE_TABLE) != 0;
  return MPL_OK;
}

// Chains per wavefront of the launch described by p (its directions filled in): the one place where
// a launch is given to the packed scans (>= 2) or to the one-chain-per-wavefront kernels (0).
// Everything that depends on that choice (the launcher, the number of wavefronts, whether the
// Jacobi scans form U themselves) reads p.pack.
template <typename Params>
int decide_pack(const mpl_shape* s, const Params& p, const CallOpts& o) {
  if (!o.packed) return 0;
  const int G = packed_chains_per_wave(s->batch, s->height, s->width, s->n_disp, s->ctx2d != 0,
                                       p.block_prefix[p.n_dirs], o.packed == 2);
  return G >= 2 ? G : 0;
}

// Wavefronts per chain for the forward scan of a launch whose caller declared a dense 1-D table
// (MPL_F_DENSE_TABLE) with several labels per lane: four (one on every SIMD of a compute unit, each
// scanning a quarter of the front labels of a pixel), two, or one.  A lone wavefront on a SIMD
// reaches some 70 % of what the SIMD issues with three of them, and the wavefronts of a chain meet
// at a barrier every pixel and repeat what is not the scan (loads, the update of the unary term,
// normalisation; the first one also finds the argmin labels), so the split pays as long as it fills
// idle SIMDs and stops paying once one wavefront per chain loads every SIMD.  Measured on 192
// labels, forward scan, ms per launch with 1 / 2 / 4 / 8 wavefronts per chain; keeping argmin
// labels: 384 chains 5.6 / 4.4 / 3.3 / 6.4, 768 chains 5.4 / 4.5 / 3.8 / 9.4, 1248 chains
// 22.7 / 18.5 / 21.3 / 50.8, 1536 chains 7.3 / 5.9 / 7.4 / 18.9, 1920 chains 8.6 / 9.6 / 10.0 / 25.1,
// 2496 chains 32.3 / 30.9 / 40.1 / 102, 3072 chains 10.2 / 12.4 / 14.3 / 37.8; without them: 384
// chains 4.5 / 2.9 / 1.9 / 3.2, 768 chains 4.1 / 2.9 / 3.2 / 4.8, 1248 chains 18.4 / 15.9 / 15.7 / 26.0,
// 1536 chains 5.9 / 6.0 / 5.6 / 9.6, 1920 chains 5.8 / 6.1 / 7.3 / 12.8, 2496 chains
// 29.9 / 27.5 / 29.2 / 51.8, 3072 chains 8.9 / 9.2 / 10.7 / 19.2.  In chains per SIMD: four
// wavefronts up to 1 (0.5 without argmin labels), two up to 1.5, one beyond.
template <typename Params>
int choose_split(const mpl_shape* s, const Params& p, const CallOpts& o, bool train) {
  if (!o.dense_table || s->ctx2d || s->n_disp <= kWave || p.pack >= 2) return 0;
  const int L = s->n_disp, R = labels_per_lane(L);
  const int forced = g_split_waves.load(std::memory_order_relaxed);
  int w;
  if (forced > 0) {
    w = forced;
  } else {
    const int64_t chains4 = 4 * (int64_t)p.block_prefix[p.n_dirs];  // in quarters of a chain
    const int64_t n_simd = launch_policy().n_simd;
    if (chains4 <= (train ? 4 : 2) * n_simd)
      w = 4;
    else if (chains4 <= 6 * n_simd)
      w = 2;
    else
      return 0;
  }
  // every wavefront needs a share of the front labels
  while (w > 1 && (w - 1) * split_share(L, R, w) >= L) --w;
  return w >= 2 ? w : 0;
}

// wavefronts of a one-direction launch: one per chain, or one per group of p.pack chains
template <typename Params>
int launch_waves(const Params& p) {
  const int chains = p.block_prefix[p.n_dirs];
  return p.pack >= 2 ? (chains + p.pack - 1) / p.pack : chains;
}

void launch_fwd(const SweepParams& p, bool train, bool jacobi, hipStream_t st) {
  Timed timed(jacobi ? MPL_KERNEL_FWD_SWEEP_ALL : MPL_KERNEL_FWD_SWEEP, st, p.fused_pair ? 2 : 1);
  if (p.pack >= 2) {
    launch_packed_fwd(p, train, jacobi, p.pack, st);  // (u_fused is never set together with pack)
    return;
  }
  switch (labels_per_lane(p.L)) {
    case 1: launch_sweep_fwd<1>(p, train, jacobi, st); break;
    case 2: launch_sweep_fwd<2>(p, train, jacobi, st); break;
    case 3: launch_sweep_fwd<3>(p, train, jacobi, st); break;
    default: launch_sweep_fwd<4>(p, train, jacobi, st); break;
  }
}

void launch_bwd(const BackParams& p, bool jacobi, hipStream_t st) {
  Timed timed(jacobi ? MPL_KERNEL_BWD_SWEEP_ALL : MPL_KERNEL_BWD_SWEEP, st, p.fused_pair ? 2 : 1);
  if (p.pack >= 2) {
    launch_packed_bwd(p, jacobi, p.pack, st);
    return;
  }
  switch (labels_per_lane(p.L)) {
    case 1: launch_sweep_bwd<1>(p, jacobi, st); break;
    case 2: launch_sweep_bwd<2>(p, jacobi, st); break;
    case 3: launch_sweep_bwd<3>(p, jacobi, st); break;
    default: launch_sweep_bwd<4>(p, jacobi, st); break;
  }
}

SweepParams base_fwd_params(const mpl_shape* s, float rho, const float* edge, const float* ctx,
                            const CtxDesc* desc) {
  SweepParams p;
  memset(&p, 0, sizeof(p));
  p.B = s->batch;
  p.H = s->height;
  p.W = s->width;
  p.L = s->n_disp;
  p.ctx2d = s->ctx2d ? 1 : 0;
  p.rho = rho;
  p.edge = edge;
  p.ctx = ctx;
  p.desc = desc;
  p.u_stride = (int64_t)s->batch * s->height * s->width * s->n_disp;
  return p;
}

// plain zero fill (a kernel, so that a caller may capture the call in a graph); V floats per store
template <int V>
__global__ void __launch_bounds__(256) zero_fill_kernel(float* __restrict__ dst, int64_t n) {
  Pack<V> z;
#pragma unroll
  for (int j = 0; j < V; ++j) z.v[j] = 0.f;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V; i < n;
       i += (int64_t)gridDim.x * blockDim.x * V)
    st_pack<V>(dst + i, z);
}

void zero_fill(float* dst, int64_t n, hipStream_t st) {
  if ((n & 3) == 0 && aligned16(dst))
    zero_fill_kernel<4><<<elementwise_blocks(n / 4), 256, 0, st>>>(dst, n);
  else
    zero_fill_kernel<1><<<elementwise_blocks(n), 256, 0, st>>>(dst, n);
}

// The sweeps keep the belief plane up to date by differences, S <- (S - m_old) + m_new, where the
// reference re-sums unary + sum_k m_k before every sweep (UpdateUnaryKernel, TRWP_forward.cu:60-80):
// the rounding of each update stays in the plane.  Between two iterations the plane holds S itself,
// so it can be re-summed there exactly as the reference sums it, which bounds the drift of long
// runs (the 50 iterations of energy minimisation) at what a few iterations accumulate.
// Iterations between two re-summations for a call (0: none).  Left to the library (-1), calls of at
// most kShortCallSweeps direction sweeps are not re-summed (what they accumulate is below the
// rounding of the reference's own fp32 sums), longer ones whenever kSweepsPerRebuild sweeps have
// passed.
constexpr int kShortCallSweeps = 64;
constexpr int kSweepsPerRebuild = 32;
int belief_rebuild_interval(int n_dir, int n_iter) {
  const int opt = g_belief_rebuild.load(std::memory_order_relaxed);
  if (opt >= 0) return opt;
  if ((int64_t)n_dir * n_iter <= kShortCallSweeps) return 0;
  return kSweepsPerRebuild / n_dir > 1 ? kSweepsPerRebuild / n_dir : 1;
}

void rebuild_belief(const mpl_shape* s, const float* unary, const float* msg, float* S,
                    hipStream_t st) {
  Timed timed(MPL_KERNEL_BELIEF, st);
  const int64_t N = (int64_t)s->batch * s->height * s->width * s->n_disp;
  const bool v4 = (N % 4 == 0) && aligned16(unary) && aligned16(msg) && aligned16(S);
  MPL_EW_LAUNCH(belief_kernel, v4, s->n_dir, N, st, unary, msg, s->n_dir, N, S, (int*)nullptr);
}

// cost_final is not written before the final aggregation, so its first bytes carry the context
// descriptor during the sweeps (no allocation, no state shared between streams).
const CtxDesc* make_desc(const mpl_shape* s, const float* ctx, float* cost_final, hipStream_t st) {
  int64_t N = (int64_t)s->batch * s->height * s->width * s->n_disp;
  if (N * (int64_t)sizeof(float) < (int64_t)sizeof(CtxDesc)) return nullptr;  // dense path
  CtxDesc* d = reinterpret_cast<CtxDesc*>(cost_final);
  Timed timed(MPL_KERNEL_OTHER, st);
  analyze_context_kernel<<<1, kWave, 0, st>>>(ctx, s->n_disp, s->ctx2d ? 1 : 0, d);
  return d;
}

}  // namespace

namespace mpl {
// SIMDs of the current device: four per compute unit.  Without a device (argument validation on a
// host that has none) the MI355X's 256 compute units are assumed.
const LaunchPolicy& launch_policy() {
  constexpr int kMaxDevices = 64;
  static LaunchPolicy table[kMaxDevices];
  static std::atomic<int> ready[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
  if (ready[dev].load(std::memory_order_acquire) == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
      (void)hipGetLastError();
      cus = 256;
    }
    LaunchPolicy pol;
    pol.n_simd = 4 * cus;
    pol.fused_pair_max_waves = pol.n_simd;
    pol.packed_min_chains = pol.n_simd + 1;
    pol.packed_min_chains21 = 2 * pol.n_simd + 1;
    pol.packed_min_chains_1d8 = 6 * pol.n_simd + 1;
    pol.packed_min_chains_1d16 = 9 * pol.n_simd + 1;
    pol.direct_max_chains = 2 * pol.n_simd;
    static std::mutex mu;
    std::lock_guard<std::mutex> lk(mu);
    if (ready[dev].load(std::memory_order_relaxed) == 0) {
      table[dev] = pol;
      ready[dev].store(1, std::memory_order_release);
    }
  }
  return table[dev];
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
}  // namespace mpl

// ------------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------------
extern "C" {

const char* mpl_last_error(void) { return g_err; }

int mpl_version(void) { return 210; }  // (2.10: the probes left the library; MPL_OPT_BELIEF_REBUILD; CPU forward)

int mpl_set_option(int option, int value) {
  if (option == MPL_OPT_PACKED_SCANS) {
    if (value < 0 || value > 2) return fail(MPL_EINVAL, "set_option: packed scans take 0, 1 or 2");
    g_packed_scans.store(value, std::memory_order_relaxed);
    return MPL_OK;
  }
  if (option == MPL_OPT_FUSED_U) {
    if (value < 0 || value > 1) return fail(MPL_EINVAL, "set_option: fused U takes 0 or 1");
    g_fused_u.store(value, std::memory_order_relaxed);
    return MPL_OK;
  }
  if (option == MPL_OPT_BELIEF_REBUILD) {
    if (value < -1) return fail(MPL_EINVAL, "set_option: the belief rebuild interval is >= -1");
    g_belief_rebuild.store(value, std::memory_order_relaxed);
    return MPL_OK;
  }
  if (option == MPL_OPT_CPU_THREADS) return set_cpu_threads(value);
  if (option == MPL_OPT_DENSE_SPLIT_WAVES) {
    if (value < 0 || value > 8) return fail(MPL_EINVAL, "set_option: 0 to 8 wavefronts per chain");
    g_split_waves.store(value, std::memory_order_relaxed);
    return MPL_OK;
  }
  return fail(MPL_EINVAL, "set_option: unknown option %d", option);
}

int mpl_profile_begin(void) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  for (auto& r : g_prof.recs) {
    g_prof.pool.push_back(r.start);
    g_prof.pool.push_back(r.stop);
  }
  g_prof.recs.clear();
  g_prof.on.store(true, std::memory_order_release);
  return MPL_OK;
}

int mpl_profile_end(mpl_kernel_stat* stats, int n_stats) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  g_prof.on.store(false, std::memory_order_release);
  for (int i = 0; i < n_stats; ++i) {
    stats[i].launches = 0;
    stats[i].total_ms = 0.0;
  }
  int rc = MPL_OK;
  for (auto& r : g_prof.recs) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(r.stop);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, r.start, r.stop);
    if (e != hipSuccess) {
      rc = fail(MPL_ELAUNCH, "profile_end: %s", hipGetErrorString(e));
    } else if (r.kind >= 0 && r.kind < n_stats) {
      stats[r.kind].launches += r.sweeps;
      stats[r.kind].total_ms += ms;
    }
    g_prof.pool.push_back(r.start);
    g_prof.pool.push_back(r.stop);
  }
  g_prof.recs.clear();
  return rc;
}

// The rule of analyze_context_kernel on a table in host memory: neither a band nor truncated linear.
int mpl_table_is_dense(const float* context, int n_disp) {
  if (!context || n_disp < 1) return -1;
  const int L = n_disp;
  const float tail = context[L - 1], c0 = context[0], slope = L >= 2 ? context[1] : 0.f;
  unsigned tail_bits;
  memcpy(&tail_bits, &tail, sizeof tail_bits);
  if ((tail_bits & 0x7fffffffu) > 0x7f800000u) return 1;  // a NaN tail: no fast path
  int last_ne = -1;
  bool below = true, lin = true;
  for (int i = 0; i < L; ++i) {
    const float v = context[i];
    if (!(v == tail)) last_ne = i;
    below = below && (v <= tail);
    lin = lin && (v == fminf(slope * (float)i, tail));
  }
  if (!below) return 1;
  const bool band = last_ne + 1 <= kMaxBandK;
  const bool linear = L >= 2 && c0 == 0.f && slope >= 0.f && lin;
  return (band || linear) ? 0 : 1;
}

int mpl_n_chains(int dir, int height, int width) {
  if (dir < 0 || dir >= kMaxDirs || height < 1 || width < 1) return -1;
  return make_dir(dir, height, width).n_chains;
}

int mpl_trwp_forward(const mpl_shape* s, unsigned flags, float rho, int n_iter,
                     int enable_min_a_dir, const float* unary, const float* context,
                     const float* edge_weights, float* msg, float* cost_final,
                     uint8_t* msg_min_index, uint8_t* msg_norm_index, float* unary_update,
                     uint8_t* label_all, void* stream) {
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  CallOpts opts;
  if ((rc = read_flags(flags, "trwp_forward", &opts)) != MPL_OK) return rc;
  const bool msg_uninit = (flags & MPL_F_MSG_UNINIT) != 0;
  if (!unary || !context || !edge_weights || !msg || !cost_final || !unary_update)
    return fail(MPL_EINVAL, "trwp_forward: null tensor pointer");
  if ((msg_min_index == nullptr) != (msg_norm_index == nullptr))
    return fail(MPL_EINVAL, "trwp_forward: msg_min_index and msg_norm_index go together");
  hipStream_t st = (hipStream_t)stream;
  const int64_t P = (int64_t)s->batch * s->height * s->width;
  const int64_t N = P * s->n_disp;
  const bool train = msg_min_index != nullptr;

  const CtxDesc* desc = make_desc(s, context, cost_final, st);
  // Messages that start at zero by declaration: S = unary, so the belief plane need not be built
  // (the first pair of sweeps reads `unary` in its place: Q = S - m_0 - m_1 = unary, too, and the
  // even sweep has nothing to store), no plane of initial messages is read (the descriptor's
  // flag stays 0), and the first sweep of every direction writes the zero of its chain starts.
  const bool uninit = msg_uninit && desc != nullptr;
  if (msg_uninit && !uninit) zero_fill(msg, (int64_t)s->n_dir * N, st);
  // The reference's contract: `msg` holds the initial messages, which its callers always clear.
  // With more labels than the packed scans take, the messages are first only looked at (n_dir
  // planes in, nothing out): when they are all zero the belief plane is not built (the kernel
  // that builds it finds the flag clear and ends) and the first pair of sweeps does what it does
  // for messages declared zero, choosing on the device (SweepParams::zero_first).
  const bool probe_zero = !uninit && desc != nullptr && s->n_disp > kPackedMaxL;
  if (!uninit) {
    Timed timed(MPL_KERNEL_BELIEF, st);
    const bool v4 = (N % 4 == 0) && aligned16(unary) && aligned16(msg) && aligned16(unary_update);
    int* flag = desc != nullptr ? &const_cast<CtxDesc*>(desc)->msg_nonzero : nullptr;
    if (probe_zero) {
      MPL_EW_LAUNCH(check_nonzero_kernel, v4, s->n_dir, N, st, msg, s->n_dir, N, flag);
      MPL_EW_LAUNCH(belief_kernel, v4, s->n_dir, N, st, unary, msg, s->n_dir, N, unary_update,
                    (int*)nullptr, (const int*)flag);
    } else {
      MPL_EW_LAUNCH(belief_kernel, v4, s->n_dir, N, st, unary, msg, s->n_dir, N, unary_update, flag);
    }
  }

  SweepParams p = base_fwd_params(s, rho, edge_weights, context, desc);
  p.belief_zero = unary;
  p.belief_out = unary_update;
  p.msg_in = msg;
  p.msg_out = msg;
  const int rebuild = belief_rebuild_interval(s->n_dir, n_iter);
  for (int it = 0; it < n_iter; ++it) {
    if (rebuild > 0 && it > 0 && it % rebuild == 0) rebuild_belief(s, unary, msg, unary_update, st);
    for (int d = 0; d < s->n_dir; ++d) {  // Gauss-Seidel over directions: TRWP_forward.cu:440-518
      fill_dirs(s, d, 1, p.dirs, p.block_prefix, &p.n_dirs);
      p.pack = decide_pack(s, p, opts);
      p.split = choose_split(s, p, opts, train);
      p.first_iter = (it == 0);
      p.pair_q = 1;
      p.belief = (uninit && it == 0 && d <= 1) ? unary : unary_update;
      p.zero_start = (uninit && it == 0) ? 1 : 0;
      p.zero_first = (probe_zero && it == 0 && d <= 1) ? 1 : 0;
      auto skip_s = [&](int dd) {
        return (((it == n_iter - 1) && (dd == s->n_dir - 1)) ||  // cost_final is re-summed
                (uninit && it == 0 && dd == 0)) ? 1 : 0;
      };
      p.skip_s_store = skip_s(d);
      // few chains: the wavefront of a chain sweeps d and then d + 1 (the same pixels in reverse)
      p.fused_pair = (opts.fused_pairs && !(d & 1) &&
                      launch_waves(p) <= launch_policy().fused_pair_max_waves) ? 1 : 0;
      p.skip_s_store2 = skip_s(d + 1);
      if (train) {
        p.idx_min = msg_min_index + (int64_t)it * s->n_dir * N;
        p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
      }
      launch_fwd(p, train, false, st);
      if (p.fused_pair) ++d;
    }
    if (label_all) {
      Timed timed(MPL_KERNEL_LABEL, st);
      launch_labels(unary, msg, s->n_dir, P, s->n_disp, 1.f, enable_min_a_dir, label_all + it * P, st);
    }
  }
  {
    Timed timed(MPL_KERNEL_AGGREGATE, st);
    const bool v4 = (N % 4 == 0) && aligned16(unary) && aligned16(msg) && aligned16(cost_final);
    MPL_EW_LAUNCH(aggregate_kernel, v4, s->n_dir, N, st, unary, msg, s->n_dir, N, 1.f,
                  enable_min_a_dir, cost_final);
  }
  return launch_ok("trwp_forward");
}

int mpl_isgmr_forward(const mpl_shape* s, unsigned flags, int enable_sgm, float rho, int n_iter,
                      int enable_min_a_dir, const float* unary, const float* context,
                      const float* edge_weights, float* msg, float* cost_final,
                      uint8_t* msg_min_index, uint8_t* msg_norm_index, float* unary_update,
                      float* msg_update, uint8_t* label_all, void* stream) {
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  CallOpts opts;
  if ((rc = read_flags(flags, "isgmr_forward", &opts)) != MPL_OK) return rc;
  const bool msg_uninit = (flags & MPL_F_MSG_UNINIT) != 0;
  if (!unary || !context || !edge_weights || !msg || !cost_final || !unary_update || !msg_update)
    return fail(MPL_EINVAL, "isgmr_forward: null tensor pointer");
  if ((msg_min_index == nullptr) != (msg_norm_index == nullptr))
    return fail(MPL_EINVAL, "isgmr_forward: msg_min_index and msg_norm_index go together");
  hipStream_t st = (hipStream_t)stream;
  const int64_t P = (int64_t)s->batch * s->height * s->width;
  const int64_t N = P * s->n_disp;
  const bool train = msg_min_index != nullptr;
  const float factor = enable_sgm ? (float)s->n_dir : 1.f;

  const CtxDesc* desc = make_desc(s, context, cost_final, st);
  SweepParams p = base_fwd_params(s, rho, edge_weights, context, desc);
  p.belief = unary_update;
  p.belief_out = nullptr;
  fill_dirs(s, 0, s->n_dir, p.dirs, p.block_prefix, &p.n_dirs);
  p.u_pair_share = (rho == 1.f) ? 1 : 0;
  // Messages that start at zero by declaration: U_d = rho * unary in the first iteration, so at
  // rho = 1 its sweeps read `unary` itself and the pass that would store U is skipped (the
  // sweeps write every element of their output buffer, chain starts included).
  const bool unary_as_u = msg_uninit && rho == 1.f;
  // Four directions at rho = 1: U of a pair of opposite directions is the unary plus the two
  // messages of the other pair, so the scans can form it on the fly (3 planes read per direction
  // instead of 1) and the pass that stores U (5 planes in, 2 out per iteration) is dropped; with
  // more directions the scans would read more than that pass moves.  (Not where the packed scans
  // of small label counts run: they are bound by the instructions of a step, and two more loads
  // per step cost them more than the pass.)
  p.pack = decide_pack(s, p, opts);
  p.split = choose_split(s, p, opts, train);
  const bool fuse_u = opts.fused_u && s->n_dir == 4 && rho == 1.f && p.pack == 0;
  if (msg_uninit && !unary_as_u) zero_fill(msg, (int64_t)s->n_dir * N, st);
  // The reference's contract at rho = 1, one chain per wavefront: the initial messages are looked
  // at first (n_dir planes in, nothing out); when they are all zero, as the reference's callers
  // pass them, the first iteration's U pass finds the flag clear and ends, and its scans read the
  // unary terms, chosen on the device (SweepParams::zero_first).
  const bool probe_zero = !msg_uninit && rho == 1.f && desc != nullptr && s->n_disp > kPackedMaxL &&
                          p.pack == 0;
  p.belief_zero = unary;
  float* have = msg;  // the buffer that holds the current messages
  for (int it = 0; it < n_iter; ++it) {
    // Jacobi over directions (ISGMR_forward.cu:506-622): every direction reads the old messages,
    // through U; the two buffers alternate instead of being copied.  U normally overwrites the
    // old messages and the new ones go to the other buffer; with an odd number of iterations the
    // first one stores U in the other buffer and the new messages in `msg`, so that the final
    // messages always end up in `msg` as in the reference.
    float* other = (have == msg) ? msg_update : msg;
    const bool out_of_place = (it == 0) && (n_iter & 1);
    float* ubuf = out_of_place ? other : have;
    float* nxt = out_of_place ? have : other;
    p.u_fused = 0;
    if (it == 0 && unary_as_u) {
      p.msg_in = unary;
      p.u_stride = 0;
    } else if (fuse_u && !out_of_place) {
      // the scans read the unary and the old messages of the other pair of directions themselves
      p.belief = unary;
      p.msg_in = have;
      p.u_stride = N;
      p.u_fused = 1;
    } else {
      Timed timed(MPL_KERNEL_UNARY_ALL, st);
      const bool v4 = (N % 4 == 0) && aligned16(unary) && aligned16(msg) && aligned16(msg_update);
      const int* only_if = nullptr;
      if (probe_zero && it == 0) {
        int* flag = &const_cast<CtxDesc*>(desc)->msg_nonzero;
        MPL_EW_LAUNCH(check_nonzero_kernel, v4, s->n_dir, N, st, have, s->n_dir, N, flag);
        only_if = flag;
        p.zero_first = 1;
      }
      MPL_EW_LAUNCH(isgmr_unary_kernel, v4, s->n_dir, N, st, unary, have, ubuf, s->n_dir, N, rho,
                    p.u_pair_share, only_if);
      p.msg_in = ubuf;
      p.u_stride = N;
    }
    p.msg_out = nxt;
    if (train) {
      p.idx_min = msg_min_index + (int64_t)it * s->n_dir * N;
      p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
    }
    launch_fwd(p, train, true, st);
    p.zero_first = 0;
    if (label_all) {
      Timed timed(MPL_KERNEL_LABEL, st);
      launch_labels(unary, nxt, s->n_dir, P, s->n_disp, factor, enable_min_a_dir, label_all + it * P, st);
    }
    have = nxt;
  }
  {
    Timed timed(MPL_KERNEL_AGGREGATE, st);
    const bool v4 = (N % 4 == 0) && aligned16(unary) && aligned16(msg) && aligned16(cost_final);
    MPL_EW_LAUNCH(aggregate_kernel, v4, s->n_dir, N, st, unary, msg, s->n_dir, N, factor,
                  enable_min_a_dir, cost_final);
  }
  return launch_ok("isgmr_forward");
}

int mpl_trwp_backward(const mpl_shape* s, unsigned flags, float rho, int n_iter,
                      const float* context, const float* edge_weights, const float* dcost_final,
                      const uint8_t* msg_min_index, const uint8_t* msg_norm_index, float* dunary,
                      float* dcontext, float* dedge_weights, float* dmsg, float* dunary_update,
                      void* stream) {
  (void)dunary_update;
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  CallOpts opts;
  if ((rc = read_flags(flags, "trwp_backward", &opts)) != MPL_OK) return rc;
  // dcontext / dedge_weights may be null: gradients the caller has no use for
  if (!context || !edge_weights || !dcost_final || !msg_min_index || !msg_norm_index || !dunary ||
      !dmsg)
    return fail(MPL_EINVAL, "trwp_backward: null tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const int64_t P = (int64_t)s->batch * s->height * s->width;
  const int64_t N = P * s->n_disp;

  BackParams p;
  memset(&p, 0, sizeof(p));
  p.B = s->batch;
  p.H = s->height;
  p.W = s->width;
  p.L = s->n_disp;
  p.ctx2d = s->ctx2d ? 1 : 0;
  p.rho = rho;
  p.a_out = dunary;
  p.h = dmsg;
  p.edge = edge_weights;
  p.ctx = context;
  p.dedge = dedge_weights;
  p.dctx = dcontext;
  p.same_label = (flags & MPL_F_DCONTEXT_SAME_LABEL) ? 1 : 0;
  bool first = true;
  for (int it = n_iter - 1; it >= 0; --it) {
    for (int d = s->n_dir - 1; d >= 0; --d) {  // TRWP_backward.cu:337-424
      fill_dirs(s, d, 1, p.dirs, p.block_prefix, &p.n_dirs);
      p.pack = decide_pack(s, p, opts);
      p.a_in = first ? dcost_final : dunary;  // CostAggregateKernelBack: every g_k starts as dcost
      p.first_touch = (it == n_iter - 1) && (d & 1);
      p.inv_from_a = (d & 1) ? 0 : 1;  // the launch before an even direction swept d + 1 = d ^ 1
      // in the last iteration walked (it == 0) the even sweeps leave h planes nobody reads again
      p.skip_hd_store = ((d & 1) || it == 0) ? 1 : 0;
      p.skip_hi_store = (!(d & 1) && it == 0) ? 1 : 0;
      p.idx_min = msg_min_index + (int64_t)it * s->n_dir * N;
      p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
      // few chains: the wavefront of a chain walks d (odd) and then d - 1 (same pixels, reversed)
      p.fused_pair = (opts.fused_pairs && (d & 1) &&
                      launch_waves(p) <= launch_policy().fused_pair_max_waves) ? 1 : 0;
      p.skip_h2 = (it == 0) ? 1 : 0;
      launch_bwd(p, false, st);
      first = false;
      if (p.fused_pair) --d;
    }
  }
  return launch_ok("trwp_backward");
}

int mpl_isgmr_backward(const mpl_shape* s, unsigned flags, int enable_sgm, float rho, int n_iter,
                       const float* context, const float* edge_weights, const float* dcost_final,
                       const uint8_t* msg_min_index, const uint8_t* msg_norm_index, float* dunary,
                       float* dcontext, float* dedge_weights, float* dmsg, float* dunary_update,
                       float* dmsg_update, void* stream) {
  (void)dunary_update;
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  CallOpts opts;
  if ((rc = read_flags(flags, "isgmr_backward", &opts)) != MPL_OK) return rc;
  // dcontext / dedge_weights may be null: gradients the caller has no use for
  if (!context || !edge_weights || !dcost_final || !msg_min_index || !msg_norm_index || !dunary ||
      !dmsg_update)
    return fail(MPL_EINVAL, "isgmr_backward: null tensor pointer");
  // The reverse scans write X_k = dU_k into dmsg_update; the recombined gradients gu_k of the next
  // (earlier) iteration go to dmsg when the caller passes it, so that at rho == 1 one plane per
  // pair of opposite directions suffices; without dmsg they overwrite X_k in place.
  {
    const int64_t planes = (int64_t)s->n_dir * s->batch * s->height * s->width * s->n_disp;
    if (dmsg != nullptr && dmsg < dmsg_update + planes && dmsg_update < dmsg + planes)
      dmsg = nullptr;  // overlaps dmsg_update: not usable as a second buffer
  }
  float* gu_buf = dmsg != nullptr ? dmsg : dmsg_update;
  const int pair_share = (dmsg != nullptr && rho == 1.f) ? 1 : 0;
  hipStream_t st = (hipStream_t)stream;
  const int64_t P = (int64_t)s->batch * s->height * s->width;
  const int64_t N = P * s->n_disp;
  const float factor = enable_sgm ? (float)s->n_dir : 1.f;

  BackParams p;
  memset(&p, 0, sizeof(p));
  p.B = s->batch;
  p.H = s->height;
  p.W = s->width;
  p.L = s->n_disp;
  p.ctx2d = s->ctx2d ? 1 : 0;
  p.rho = rho;
  p.du_out = dmsg_update;
  p.edge = edge_weights;
  p.ctx = context;
  p.dedge = dedge_weights;
  p.dctx = dcontext;
  p.same_label = (flags & MPL_F_DCONTEXT_SAME_LABEL) ? 1 : 0;
  fill_dirs(s, 0, s->n_dir, p.dirs, p.block_prefix, &p.n_dirs);
  p.pack = decide_pack(s, p, opts);
  for (int it = n_iter - 1; it >= 0; --it) {
    const bool first = (it == n_iter - 1);
    p.gu_in = first ? dcost_final : gu_buf;  // gu_k = dcost_final for every k at the start
    p.gu_stride = first ? 0 : N;
    p.gu_pair_share = first ? 0 : pair_share;
    p.idx_min = msg_min_index + (int64_t)it * s->n_dir * N;
    p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
    launch_bwd(p, true, st);
    Timed timed(MPL_KERNEL_COMBINE, st);
    const bool v4 = (N % 4 == 0) && aligned16(dmsg_update) && aligned16(gu_buf) &&
                    aligned16(dcost_final) && aligned16(dunary);
    MPL_EW_LAUNCH(isgmr_combine_kernel, v4, s->n_dir, N, st, dmsg_update, gu_buf, s->n_dir, N, rho,
                  dcost_final, factor, first ? 1 : 0, it > 0 ? 1 : 0, pair_share, dunary);
  }
  return launch_ok("isgmr_backward");
}

// ---- soft-weighted TRWP ------------------------------------------------------------------------
int mpl_trwp_soft_forward(const mpl_shape* s, unsigned flags, float rho, int n_iter,
                          const float* unary, const float* context, const float* edge_weights,
                          float* msg, float* msg_edge_label, uint8_t* msg_norm_index,
                          float* cost_final, float* unary_update, uint8_t* label_all,
                          void* stream) {
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  CallOpts opts;
  if ((rc = read_flags(flags, "trwp_soft_forward", &opts)) != MPL_OK) return rc;
  if (!unary || !context || !edge_weights || !msg || !cost_final || !unary_update)
    return fail(MPL_EINVAL, "trwp_soft_forward: null tensor pointer");
  if ((msg_edge_label == nullptr) != (msg_norm_index == nullptr))
    return fail(MPL_EINVAL, "trwp_soft_forward: msg_edge_label and msg_norm_index go together");
  hipStream_t st = (hipStream_t)stream;
  const int64_t P = (int64_t)s->batch * s->height * s->width;
  const int64_t N = P * s->n_disp;
  const bool train = msg_edge_label != nullptr;
  if (flags & MPL_F_MSG_UNINIT) zero_fill(msg, (int64_t)s->n_dir * N, st);
  {
    Timed timed(MPL_KERNEL_BELIEF, st);
    const bool v4 = (N % 4 == 0) && aligned16(unary) && aligned16(msg) && aligned16(unary_update);
    MPL_EW_LAUNCH(belief_kernel, v4, s->n_dir, N, st, unary, msg, s->n_dir, N, unary_update,
                  (int*)nullptr);
  }
  SweepParams p = base_fwd_params(s, rho, edge_weights, context, nullptr);
  p.belief = unary_update;
  p.belief_out = unary_update;
  p.msg_in = msg;
  p.msg_out = msg;
  const int rebuild = belief_rebuild_interval(s->n_dir, n_iter);
  for (int it = 0; it < n_iter; ++it) {
    if (rebuild > 0 && it > 0 && it % rebuild == 0) rebuild_belief(s, unary, msg, unary_update, st);
    for (int d = 0; d < s->n_dir; ++d) {  // TRWP_forward_soft.cu:441-520
      fill_dirs(s, d, 1, p.dirs, p.block_prefix, &p.n_dirs);
      if (train) {
        p.edge_label = msg_edge_label + (int64_t)it * s->n_dir * N * s->n_disp;
        p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
      }
      // few chains of at most 32 labels: the wavefront of a chain sweeps d and then d + 1
      p.fused_pair = (opts.fused_pairs && s->n_disp <= 32 &&
                      p.block_prefix[p.n_dirs] <= launch_policy().fused_pair_max_waves) ? 1 : 0;
      Timed timed(MPL_KERNEL_FWD_SWEEP, st, p.fused_pair ? 2 : 1);
      launch_soft_fwd(p, train, st);
      if (p.fused_pair) ++d;
    }
    if (label_all) {
      Timed timed(MPL_KERNEL_LABEL, st);
      launch_labels(unary, msg, s->n_dir, P, s->n_disp, 1.f, 0, label_all + it * P, st);
    }
  }
  {
    Timed timed(MPL_KERNEL_AGGREGATE, st);
    const bool v4 = (N % 4 == 0) && aligned16(unary) && aligned16(msg) && aligned16(cost_final);
    MPL_EW_LAUNCH(aggregate_kernel, v4, s->n_dir, N, st, unary, msg, s->n_dir, N, 1.f, 0,
                  cost_final);
  }
  return launch_ok("trwp_soft_forward");
}

int mpl_trwp_soft_backward(const mpl_shape* s, unsigned flags, float rho, int n_iter,
                           const float* dcost_final, const float* context,
                           const float* edge_weights, const float* msg_edge_label,
                           const uint8_t* msg_norm_index, float* dunary, float* dcontext,
                           float* dedge_weights, float* dmsg, float* dunary_update, void* stream) {
  (void)dunary_update;
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  CallOpts opts;
  if ((rc = read_flags(flags, "trwp_soft_backward", &opts)) != MPL_OK) return rc;
  if (!context || !edge_weights || !dcost_final || !msg_edge_label || !msg_norm_index || !dunary ||
      !dmsg)
    return fail(MPL_EINVAL, "trwp_soft_backward: null tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const int64_t P = (int64_t)s->batch * s->height * s->width;
  const int64_t N = P * s->n_disp;
  BackParams p;
  memset(&p, 0, sizeof(p));
  p.B = s->batch;
  p.H = s->height;
  p.W = s->width;
  p.L = s->n_disp;
  p.ctx2d = s->ctx2d ? 1 : 0;
  p.rho = rho;
  p.a_out = dunary;
  p.h = dmsg;
  p.edge = edge_weights;
  p.ctx = context;
  p.dedge = dedge_weights;
  p.dctx = dcontext;
  bool first = true;
  for (int it = n_iter - 1; it >= 0; --it) {
    for (int d = s->n_dir - 1; d >= 0; --d) {  // TRWP_backward_soft.cu:454-538
      fill_dirs(s, d, 1, p.dirs, p.block_prefix, &p.n_dirs);
      p.a_in = first ? dcost_final : dunary;
      p.first_touch = (it == n_iter - 1) && (d & 1);
      p.edge_label = msg_edge_label + (int64_t)it * s->n_dir * N * s->n_disp;
      p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
      // few chains of at most 32 labels: the wavefront of a chain walks d (odd) and then d - 1
      p.fused_pair = (opts.fused_pairs && s->n_disp <= 32 &&
                      p.block_prefix[p.n_dirs] <= launch_policy().fused_pair_max_waves) ? 1 : 0;
      Timed timed(MPL_KERNEL_BWD_SWEEP, st, p.fused_pair ? 2 : 1);
      launch_soft_bwd(p, st);
      first = false;
      if (p.fused_pair) --d;
    }
  }
  return launch_ok("trwp_soft_backward");
}

int mpl_soft_weighted_message(int n_trees, int n_disp, const float* message,
                              float* message_soft_sum_norm, uint8_t* message_soft_sum_min_ind,
                              void* stream) {
  if (n_trees < 0 || n_disp < 1 || n_disp > kMaxL)
    return fail(MPL_EINVAL, "soft_weighted_message: n_trees >= 0 and 1 <= n_disp <= %d needed", kMaxL);
  if (!message || !message_soft_sum_norm || !message_soft_sum_min_ind)
    return fail(MPL_EINVAL, "soft_weighted_message: null tensor pointer");
  launch_swm_fwd(message, n_trees, n_disp, message_soft_sum_norm, message_soft_sum_min_ind,
                 (hipStream_t)stream);
  return launch_ok("soft_weighted_message");
}

int mpl_soft_weighted_message_back(int n_trees, int n_disp, const float* dmessage_soft_sum_norm,
                                   const float* message, const uint8_t* message_soft_sum_min_ind,
                                   float* dmessage, void* stream) {
  if (n_trees < 0 || n_disp < 1 || n_disp > kMaxL)
    return fail(MPL_EINVAL, "soft_weighted_message_back: n_trees >= 0 and 1 <= n_disp <= %d needed",
                kMaxL);
  if (!dmessage_soft_sum_norm || !message || !message_soft_sum_min_ind || !dmessage)
    return fail(MPL_EINVAL, "soft_weighted_message_back: null tensor pointer");
  launch_swm_bwd(dmessage_soft_sum_norm, message, message_soft_sum_min_ind, n_trees, n_disp,
                 dmessage, (hipStream_t)stream);
  return launch_ok("soft_weighted_message_back");
}

}  // extern "C"
