/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the TRWP / ISGMR message-passing path.
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may load this.
 *
 * Part 1: geometry shared by every restated kernel (common.cpp:17-103 and the chain
 *         start computations of the scan kernels).
 * Part 2: the GPU-kernel semantics (mp_oracle_impl.h, instantiated for float and double).
 * Part 3: the reference's CPU forward path restated with its own loop nest
 *         (TRWP.cpp:10-243, ISGMR.cpp:10-298, common.cpp:105-161): no edge weights, no
 *         indices, messages re-summed inside the innermost loop, OpenMP over chains.
 *         It is what the benchmark times as the CPU baseline.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC mp_oracle.c -o libmp_oracle.so -lm
 * (-ffp-contract=off: the source order of every multiply and add is kept as written.)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
  int n_dir, B, H, W, L; /* B = batch * n_cv */
  int ctx2d;             /* 1: (L,L) table read at [min*L+max]; the reference ties this to L == 21 */
} mpo_geom;

static inline int64_t mpo_pixels(const mpo_geom* g) { return (int64_t)g->B * g->H * g->W; }
static inline int64_t mpo_plane(const mpo_geom* g) { return mpo_pixels(g) * g->L; }

/* direction table: common.cpp:28-76 */
void mpo_dir_step(int dir, int* hs, int* ws) {
  static const int tab[16][2] = {{0, 1},  {0, -1}, {1, 0},  {-1, 0},  {1, 1},  {-1, -1},
                                 {1, -1}, {-1, 1}, {1, 2},  {-1, -2}, {2, 1},  {-2, -1},
                                 {2, -1}, {-2, 1}, {1, -2}, {-1, 2}};
  *hs = tab[dir][0];
  *ws = tab[dir][1];
}

/* number of chains ("trees") per direction: common.cpp:78-87 */
int mpo_n_trees(int dir, int H, int W) {
  int hs, ws;
  mpo_dir_step(dir, &hs, &ws);
  if (dir <= 1) return H;
  if (dir <= 3) return W;
  if (dir <= 7) return H + W - 1;
  int ha = abs(hs), wa = abs(ws);
  return ha > wa ? H + (W - 1) * ha : W + (H - 1) * wa;
}

/*
 * Start pixel and loop count of one chain.  (hs, ws) is the step the scan walks with, i.e.
 * already negated for the backward kernels.  Which formula applies depends on the kernel the
 * reference launches for `dir`: Horizontal for 0-1 (TRWP_forward.cu:107-110), DiagonalNarrow
 * when |h_step| > |w_step| (:200-218), DiagonalWide otherwise (:308-313).
 */
void mpo_tree_start(int dir, int hs, int ws, int H, int W, int tree, int* h0, int* w0,
                    int* n_roll) {
  int ha = abs(hs), wa = abs(ws);
  if (dir < 2) {
    *h0 = tree;
    *w0 = ws > 0 ? 0 : W - 1;
    *n_roll = W - 1;
    return;
  }
  int shift = tree - (H - 1) * (ws > 0 ? ws : 0);
  if (ha > wa) {
    /* `int % uint` in the reference: the dividend is converted to unsigned first */
    int common1 = (int)((unsigned)shift % (unsigned)ha);
    float common2 = (float)shift / (float)ha;
    int hstart, wstart;
    if (ws > 0) {
      hstart = (ha - common1) % ha;
      wstart = (int)ceilf(common2);
    } else {
      hstart = common1;
      wstart = (int)floorf(common2);
    }
    if (hs < 0) hstart = H - 1 - hstart;
    *h0 = hstart;
    *w0 = wstart;
    *n_roll = (H - 1) / ha;
    return;
  }
  *h0 = hs > 0 ? 0 : H - 1;
  *w0 = shift;
  *n_roll = (H - 1) / ha;
}

#define MPO_CAT2(a, b) a##b
#define MPO_CAT(a, b) MPO_CAT2(a, b)

#define REAL float
#define FN(name) MPO_CAT(name, _f32)
#include "mp_oracle_impl.h"
#undef REAL
#undef FN

#define REAL double
#define FN(name) MPO_CAT(name, _f64)
#include "mp_oracle_impl.h"
#undef REAL
#undef FN

/* ===== Part 3: the reference's CPU forward path, loop nest kept ============================ */

#define REF_NUM_THREADS 16 /* tools/cpp/utils.h:17 */

/* DynamicProgramming: TRWP.cpp:10-84 / ISGMR.cpp:10-95.  msg_self is the plane the chain reads its
 * own direction from and writes to: msg[dir] for TRWP (in place), msg_update[dir] for ISGMR. */
static void refcpu_chain(const mpo_geom* g, int dir, int hs, int ws, float rho, int64_t bv_off,
                         int h0, int w0, int n_roll, const float* unary, const float* msg,
                         float* msg_self, const float* context) {
  int L = g->L, H = g->H, W = g->W, n_dir = g->n_dir, inv = dir ^ 1;
  int64_t N = mpo_plane(g);
  for (int i = 0; i <= n_roll; ++i) {
    int ch = h0 + i * hs, cw = w0 + i * ws, fh = ch - hs, fw = cw - ws;
    if (ch < 0 || ch >= H || fh < 0 || fh >= H || cw < 0 || cw >= W || fw < 0 || fw >= W) continue;
    int64_t fbase = bv_off + ((int64_t)fh * W + fw) * L;
    int64_t cbase = bv_off + ((int64_t)ch * W + cw) * L;
    float norm_min = 0;
    for (int cd = L - 1; cd >= 0; --cd) {
      float min_value = 0;
      for (int fd = L - 1; fd >= 0; --fd) {
        float cv;
        if (g->ctx2d) {
          int lo = cd < fd ? cd : fd, hi = cd < fd ? fd : cd;
          cv = context[(int64_t)lo * L + hi];
        } else {
          cv = context[abs(cd - fd)];
        }
        int64_t off = fbase + fd;
        float msg_sum = 0;
        for (int k = 0; k < n_dir; ++k)
          msg_sum += (k == dir) ? msg_self[off] : msg[(int64_t)k * N + off];
        float value = rho * (unary[off] + msg_sum) - msg[(int64_t)inv * N + off] + cv;
        if (fd == L - 1 || value < min_value) min_value = value;
      }
      msg_self[cbase + cd] = min_value;
      if (cd == L - 1 || min_value < norm_min) norm_min = min_value;
    }
    for (int cd = L - 1; cd >= 0; --cd) msg_self[cbase + cd] -= norm_min;
  }
}

/* Horizontal/DiagonalWide/DiagonalNarrow: TRWP.cpp:86-170 (OpenMP over chains, batch serial).
 * The reference's Horizontal passes roll_step = width, one step more than the kernels; the
 * extra step is always out of the image, so W-1 is used here. */
static void refcpu_sweep(const mpo_geom* g, int dir, float rho, const float* unary,
                         const float* msg, float* msg_self, const float* context, int n_threads) {
  int hs, ws;
  mpo_dir_step(dir, &hs, &ws);
  int n_trees = mpo_n_trees(dir, g->H, g->W);
  for (int bv = 0; bv < g->B; ++bv) {
    int64_t bv_off = (int64_t)bv * g->H * g->W * g->L;
#pragma omp parallel for schedule(dynamic) num_threads(n_threads)
    for (int tree = 0; tree < n_trees; ++tree) {
      int h0, w0, n_roll;
      mpo_tree_start(dir, hs, ws, g->H, g->W, tree, &h0, &w0, &n_roll);
      refcpu_chain(g, dir, hs, ws, rho, bv_off, h0, w0, n_roll, unary, msg, msg_self, context);
    }
  }
}

/* CostAggregate: common.cpp:105-137 */
static void refcpu_aggregate(const mpo_geom* g, const float* unary, const float* msg, float* cost,
                             int n_threads) {
  int64_t N = mpo_plane(g);
#pragma omp parallel for schedule(static) num_threads(n_threads)
  for (int64_t i = 0; i < N; ++i) {
    float s = 0;
    for (int k = 0; k < g->n_dir; ++k) s += msg[(int64_t)k * N + i] / 1.0f;
    cost[i] = unary[i] + s;
  }
}

/* ForwardCPU: TRWP.cpp:172-243.  context_stride = L*L in the reference (a (n_dir,L,L) table,
 * `context + dir*L*L`); 0 shares one table between directions. */
int mpo_refcpu_trwp_forward(const mpo_geom* g, float rho, int n_iter, const float* unary,
                            const float* context, int64_t context_stride, float* msg,
                            float* cost_final, int n_threads) {
  if (n_threads <= 0) n_threads = REF_NUM_THREADS;
  int64_t N = mpo_plane(g);
  for (int it = 0; it < n_iter; ++it)
    for (int d = 0; d < g->n_dir; ++d)
      refcpu_sweep(g, d, rho, unary, msg, msg + (int64_t)d * N, context + d * context_stride,
                   n_threads);
  refcpu_aggregate(g, unary, msg, cost_final, n_threads);
  return 0;
}

/* ForwardCPU: ISGMR.cpp:190-298 with enable_sgm == 0 */
int mpo_refcpu_isgmr_forward(const mpo_geom* g, float rho, int n_iter, const float* unary,
                             const float* context, int64_t context_stride, float* msg,
                             float* msg_update, float* cost_final, int n_threads) {
  if (n_threads <= 0) n_threads = REF_NUM_THREADS;
  int64_t N = mpo_plane(g);
  for (int it = 0; it < n_iter; ++it) {
    for (int d = 0; d < g->n_dir; ++d)
      refcpu_sweep(g, d, rho, unary, msg, msg_update + (int64_t)d * N,
                   context + d * context_stride, n_threads);
    memcpy(msg, msg_update, sizeof(float) * N * g->n_dir);
  }
  refcpu_aggregate(g, unary, msg_update, cost_final, n_threads);
  return 0;
}

int mpo_geom_size(void) { return (int)sizeof(mpo_geom); }
