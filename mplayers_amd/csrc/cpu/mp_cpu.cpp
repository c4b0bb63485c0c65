// CPU forward of TRWP and ISGMR: what the reference's operators run for tensors that are not on the
// GPU (ForwardCPU, MPLayers/TRWP/TRWP.cpp:172-243 and MPLayers/ISGMR/ISGMR.cpp:190-298, reached
// from Forward at TRWP.cpp:275-282 / ISGMR.cpp:330-339).  Host code only, compiled with the host
// compiler and linked into libmplayers_hip.so; host pointers in, host pointers out.
//
// Semantics of that path, which differ from the GPU kernels' and are reproduced bit for bit:
//   * no edge weights (every edge has weight 1) and no argmin indices: forward only;
//   * the pairwise table of direction d is read at `context + d * L * L` (TRWP.cpp:205,
//     ISGMR.cpp:226): an (n_dir, L, L) buffer, of which a 2-D table uses [min(a,b) * L + max(a,b)]
//     and a 1-D table the first L entries of each block;
//   * per edge and label pair  value = rho * (unary[q, fd] + sum_k m_k[q, fd]) - m_inv[q, fd] + ctx
//     in exactly that order (TRWP.cpp:56-60), with the messages summed in direction order from 0;
//     the message of the swept direction at q is the one the sweep has just written (TRWP sweeps
//     in place; ISGMR writes a second buffer and reads its own new message from it, :62-68);
//   * strict `<` scans from the last label down (largest label wins ties), minimum subtracted;
//   * cost_final = unary + (sum_k m_k) with the sum formed first (CostAggregate, common.cpp:105-133);
//   * labels: smallest label among equal costs, and always 0 for 256 labels, because the
//     reference's loop counter is an unsigned char compared with (uchar)256 == 0 (common.cpp:152);
//   * the SGM flag of ISGMR reads the unary term at the current pixel and label instead of the
//     front one, and after every iteration REPLACES the caller's unary tensor by the sum of the new
//     messages and clears the messages (ISGMR.cpp:255-261): `unary` is an in/out argument there.
// What is not reproduced: the reference recomputes sum_k m_k[q, fd] for every label pair
// (O(L^2 n_dir) per edge); here it is formed once per front label, which gives the same bits.
// Chains are independent (a sweep writes only the swept direction's plane, each pixel from one
// chain), so they are spread over threads as the reference spreads its trees over OpenMP threads.

#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <exception>
#include <stdexcept>
#include <thread>
#include <vector>

#include "../../../include/mplayers_amd.h"

namespace mpl {
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
}

namespace {

std::atomic<int> g_cpu_threads{0};  // MPL_OPT_CPU_THREADS; 0: the reference's 16

int n_threads() {
  const int t = g_cpu_threads.load(std::memory_order_relaxed);
  return t > 0 ? t : 16;  // NUM_THREADS, tools/cpp/utils.h:17
}

// fn(i) for i in [0, n), work handed out one block at a time (schedule(dynamic) of the reference)
template <typename Fn>
void parallel_for(int64_t n, int64_t block, const Fn& fn) {
  const int64_t n_blocks = (n + block - 1) / block;
  // (no more threads than the host has hardware threads: the results do not depend on the count)
  const int hw = (int)std::thread::hardware_concurrency();
  const int workers = (int)std::min<int64_t>(std::min(n_threads(), hw > 0 ? hw : 1), n_blocks);
  std::atomic<int64_t> next{0};
  std::atomic<bool> failed{false};
  auto body = [&]() {
    try {
      for (;;) {
        const int64_t b = next.fetch_add(1, std::memory_order_relaxed);
        if (b >= n_blocks) return;
        const int64_t end = std::min(n, (b + 1) * block);
        for (int64_t i = b * block; i < end; ++i) fn(i);
      }
    } catch (...) {  // (an allocation the host refused: reported by the calling thread)
      failed.store(true, std::memory_order_relaxed);
    }
  };
  std::vector<std::thread> pool;
  try {
    if (workers > 1) pool.reserve(workers - 1);
    for (int t = 1; t < workers; ++t) pool.emplace_back(body);
  } catch (...) {
    // fewer threads than asked for: the ones that started, and this one, do all the work
  }
  body();
  for (auto& th : pool) th.join();
  if (failed.load(std::memory_order_relaxed)) throw std::runtime_error("a worker thread failed");
}

// direction table of MPLayers/common.cpp:28-76
void dir_step(int dir, int* hs, int* ws) {
  static const int tab[16][2] = {{0, 1},  {0, -1}, {1, 0},  {-1, 0},  {1, 1},  {-1, -1}, {1, -1}, {-1, 1},
                                 {1, 2},  {-1, -2}, {2, 1}, {-2, -1}, {2, -1}, {-2, 1},  {1, -2}, {-1, 2}};
  *hs = tab[dir][0];
  *ws = tab[dir][1];
}

struct Grid {
  int n_dir, B, H, W, L, ctx2d;
  int64_t P, N;  // pixels and elements of one plane
};

// Every chain of direction `dir`: the pixels whose front neighbour lies outside the image.  These
// are the starts of the walks of the reference's trees (common.cpp:78-87, TRWP.cpp:94-167).
std::vector<int> chain_starts(const Grid& g, int hs, int ws) {
  std::vector<int> s;
  for (int h = 0; h < g.H; ++h)
    for (int w = 0; w < g.W; ++w) {
      const int fh = h - hs, fw = w - ws;
      if (fh < 0 || fh >= g.H || fw < 0 || fw >= g.W) s.push_back(h * g.W + w);
    }
  return s;
}

inline float ctx_at(const float* ctx, int L, int ctx2d, int cd, int fd) {
  return ctx2d ? ctx[(cd < fd ? cd : fd) * L + (cd < fd ? fd : cd)] : ctx[cd < fd ? fd - cd : cd - fd];
}

// One sweep of direction `dir` over every chain of every batch item.
//   m_all:   the (n_dir, N) planes the sum over directions reads (old messages)
//   m_dir:   the plane that is read at the front pixel for k == dir and written at the current one
//            (TRWP: m_all's own plane, in place; ISGMR: the plane of `dir` in the second buffer)
//   sgm:     the unary term is taken at the current pixel and label (ISGMR.cpp:72-77)
void sweep(const Grid& g, int dir, float rho, const float* unary, const float* m_all, float* m_dir,
           const float* ctx, bool sgm) {
  int hs, ws;
  dir_step(dir, &hs, &ws);
  const int inv = dir ^ 1;
  const int L = g.L;
  const std::vector<int> starts = chain_starts(g, hs, ws);
  const int64_t n_chains = (int64_t)starts.size();
  // the table as ctx(cd, fd) rows, so that the scan over fd reads consecutive floats
  std::vector<float> tab((size_t)L * L);
  for (int cd = 0; cd < L; ++cd)
    for (int fd = 0; fd < L; ++fd) tab[(size_t)cd * L + fd] = ctx_at(ctx, L, g.ctx2d, cd, fd);
  const int64_t HW = (int64_t)g.H * g.W;
  parallel_for((int64_t)g.B * n_chains, 1, [&](int64_t job) {
    const int64_t bv = job / n_chains;
    const int start = starts[(size_t)(job - bv * n_chains)];
    int h = start / g.W, w = start - (start / g.W) * g.W;
    thread_local std::vector<float> scratch;
    if (scratch.size() < 3 * (size_t)L) scratch.resize(3 * (size_t)L);
    float* base = scratch.data();
    float* sum = base + L;
    float* out = sum + L;
    for (;;) {
      const int fh = h, fw = w;
      h += hs;
      w += ws;
      if (h < 0 || h >= g.H || w < 0 || w >= g.W) break;
      const int64_t q = (bv * HW + (int64_t)fh * g.W + fw) * L;
      const int64_t p = (bv * HW + (int64_t)h * g.W + w) * L;
      for (int fd = 0; fd < L; ++fd) {
        float s = 0.f;
        for (int k = 0; k < g.n_dir; ++k) s += (k == dir) ? m_dir[q + fd] : m_all[(int64_t)k * g.N + q + fd];
        sum[fd] = s;
        if (!sgm) base[fd] = rho * (unary[q + fd] + s) - m_all[(int64_t)inv * g.N + q + fd];
      }
      float norm = 0.f;
      for (int cd = L - 1; cd >= 0; --cd) {
        const float* row = &tab[(size_t)cd * L];
        if (sgm) {
          const float u = unary[p + cd];
          for (int fd = 0; fd < L; ++fd) base[fd] = rho * (u + sum[fd]) - m_all[(int64_t)inv * g.N + q + fd];
        }
        float best = base[L - 1] + row[L - 1];
        for (int fd = L - 2; fd >= 0; --fd) {
          const float v = base[fd] + row[fd];
          best = v < best ? v : best;
        }
        out[cd] = best;
        norm = (cd == L - 1 || best < norm) ? best : norm;
      }
      for (int cd = 0; cd < L; ++cd) m_dir[p + cd] = out[cd] - norm;
    }
  });
}

// cost[i] = base[i] + (sum_k m_k[i] / 1)  (CostAggregate, common.cpp:105-133, called with the
// parameters of direction 0, whose dir_weight is 1); base may be null: zeros
void aggregate(const Grid& g, const float* base, const float* msg, float* cost) {
  parallel_for(g.P, 1024, [&](int64_t pix) {
    for (int d = 0; d < g.L; ++d) {
      const int64_t i = pix * g.L + d;
      float s = 0.f;
      for (int k = 0; k < g.n_dir; ++k) s += msg[(int64_t)k * g.N + i] / 1.f;
      cost[i] = (base != nullptr ? base[i] : 0.f) + s;
    }
  });
}

// CalLabel, common.cpp:135-161
void labels(const Grid& g, const float* cost, uint8_t* label) {
  const int n_scan = (int)(uint8_t)g.L;  // the reference's `uchar l < (uchar)n_disp`: 0 for 256 labels
  parallel_for(g.P, 1024, [&](int64_t pix) {
    const float* c = cost + pix * g.L;
    uint8_t arg = 0;
    float best = c[0];
    for (int l = 0; l < n_scan; ++l)
      if (c[l] < best) {
        best = c[l];
        arg = (uint8_t)l;
      }
    label[pix] = arg;
  });
}

int check_cpu_shape(const mpl_shape* s, int n_iter, Grid* g) {
  if (s == nullptr) return mpl::fail(MPL_EINVAL, "shape is null");
  if (s->n_dir < 2 || s->n_dir > MPL_MAX_DIRS || (s->n_dir & 1))
    return mpl::fail(MPL_EINVAL, "n_dir must be even and in [2, %d], got %d", MPL_MAX_DIRS, s->n_dir);
  if (s->batch < 1 || s->height < 1 || s->width < 1)
    return mpl::fail(MPL_EINVAL, "batch/height/width must be positive, got %d/%d/%d", s->batch,
                     s->height, s->width);
  if (s->n_disp < 1 || s->n_disp > MPL_MAX_LABELS)
    return mpl::fail(MPL_EINVAL, "n_disp must be in [1, %d], got %d", MPL_MAX_LABELS, s->n_disp);
  if (n_iter < 1) return mpl::fail(MPL_EINVAL, "n_iter must be positive, got %d", n_iter);
  if ((int64_t)s->batch * s->height * s->width > 0x7fffffff)
    return mpl::fail(MPL_EINVAL, "more than 2^31 pixels");
  g->n_dir = s->n_dir;
  g->B = s->batch;
  g->H = s->height;
  g->W = s->width;
  g->L = s->n_disp;
  g->ctx2d = s->ctx2d ? 1 : 0;
  g->P = (int64_t)s->batch * s->height * s->width;
  g->N = g->P * s->n_disp;
  return MPL_OK;
}

}  // namespace

namespace mpl {
int set_cpu_threads(int n) {
  if (n < 0 || n > 1024) return fail(MPL_EINVAL, "set_option: CPU threads must be in [0, 1024]");
  g_cpu_threads.store(n, std::memory_order_relaxed);
  return MPL_OK;
}
}  // namespace mpl

extern "C" {

int mpl_trwp_forward_cpu(const mpl_shape* shape, float rho, int n_iter, const float* unary,
                         const float* context, float* msg, float* cost_final, uint8_t* label_all) {
  Grid g;
  int rc = check_cpu_shape(shape, n_iter, &g);
  if (rc) return rc;
  if (!unary || !context || !msg || !cost_final)
    return mpl::fail(MPL_EINVAL, "trwp_forward_cpu: null tensor pointer");
  const int64_t LL = (int64_t)g.L * g.L;
  try {  // (a thread or an allocation the host refuses must not unwind through the C boundary)
    for (int it = 0; it < n_iter; ++it) {
      for (int d = 0; d < g.n_dir; ++d)  // in place, one direction after the other: TRWP.cpp:210-228
        sweep(g, d, rho, unary, msg, msg + (int64_t)d * g.N, context + d * LL, false);
      if (label_all != nullptr) {
        aggregate(g, unary, msg, cost_final);
        labels(g, cost_final, label_all + (int64_t)it * g.P);
      }
    }
    aggregate(g, unary, msg, cost_final);
  } catch (const std::exception& e) {
    return mpl::fail(MPL_ELAUNCH, "trwp_forward_cpu: %s", e.what());
  }
  return MPL_OK;
}

int mpl_isgmr_forward_cpu(const mpl_shape* shape, int enable_sgm, float rho, int n_iter,
                          float* unary, const float* context, float* msg, float* cost_final,
                          float* msg_update, uint8_t* label_all) {
  Grid g;
  int rc = check_cpu_shape(shape, n_iter, &g);
  if (rc) return rc;
  if (!unary || !context || !msg || !cost_final || !msg_update)
    return mpl::fail(MPL_EINVAL, "isgmr_forward_cpu: null tensor pointer");
  const int64_t LL = (int64_t)g.L * g.L;
  const size_t all = (size_t)g.n_dir * (size_t)g.N * sizeof(float);
  try {
    for (int it = 0; it < n_iter; ++it) {
      for (int d = 0; d < g.n_dir; ++d)  // every direction from the old messages: ISGMR.cpp:232-251
        sweep(g, d, rho, unary, msg, msg_update + (int64_t)d * g.N, context + d * LL, enable_sgm != 0);
      memcpy(msg, msg_update, all);
      if (enable_sgm) {
        aggregate(g, nullptr, msg_update, unary);  // the unary terms become the sum of the messages
        memset(msg, 0, all);
        if (label_all != nullptr) {
          memcpy(cost_final, unary, (size_t)g.N * sizeof(float));
          labels(g, cost_final, label_all + (int64_t)it * g.P);
        }
      } else if (label_all != nullptr) {
        aggregate(g, unary, msg_update, cost_final);
        labels(g, cost_final, label_all + (int64_t)it * g.P);
      }
    }
    if (enable_sgm)
      memcpy(cost_final, unary, (size_t)g.N * sizeof(float));
    else
      aggregate(g, unary, msg_update, cost_final);
  } catch (const std::exception& e) {
    return mpl::fail(MPL_ELAUNCH, "isgmr_forward_cpu: %s", e.what());
  }
  return MPL_OK;
}

}  // extern "C"
