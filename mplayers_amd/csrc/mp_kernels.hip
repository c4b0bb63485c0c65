// Min-sum message passing (TRWP / ISGMR) on grid MRFs, hand-written for gfx950 (CDNA4, wave64).
//
// Mapping: one 64-lane wavefront walks one chain (a row, column or diagonal segment) of one
// direction.  The L labels of a pixel are spread over the lanes in blocks: lane i owns labels
// R*i .. R*i+R-1 with R = ceil(L/64), so a pixel's label vector is one coalesced R-dword load per
// lane, the recurrence state (previous message) never leaves registers, a one-label shift costs a
// single DPP wave shift, and the min over labels is a DPP reduction.  Pixel data does not depend
// on the recurrence, so it is prefetched a few pixels ahead through a register ring.
//
// Traffic model: instead of re-summing all messages for every sweep (UpdateUnaryKernel of the
// reference, TRWP_forward.cu:60-80), a belief plane S = unary + sum_k m_k is kept, so a sweep of
// direction d reads S, m_d, m_inv and writes m_d (and S for TRWP): 20 B per label.  The backward
// pass keeps the gradient planes as g_k = A + h_k with one shared plane A (which ends up being
// dunary) for the same reason.
//
// Semantics follow the reference GPU kernels (cited per function); tie rules: largest front label
// for the message argmin, largest label for the normalisation argmin, smallest label for labels.

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/mplayers_amd.h"

namespace {

constexpr int kWave = 64;
constexpr int kMaxL = MPL_MAX_LABELS;
constexpr int kMaxDirs = MPL_MAX_DIRS;
constexpr int kMaxCtx2dL = 64;                       // (L,L) table kept in LDS
constexpr int kMaxBandK = 32;                        // widest band handled by the O(L*K) path
constexpr int kPrefetch = 4;                         // pixels in flight per wave

// ------------------------------------------------------------------------------------------------
// wavefront primitives
// ------------------------------------------------------------------------------------------------
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf>
__device__ __forceinline__ float dpp_f(float old, float src) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src),
                                         CTRL, ROW_MASK, BANK_MASK, false));
}
// lane i <- lane i+1 (lane 63 <- fill)
__device__ __forceinline__ float wave_shl1(float x, float fill) { return dpp_f<0x130>(fill, x); }
// lane i <- lane i-1 (lane 0 <- fill)
__device__ __forceinline__ float wave_shr1(float x, float fill) { return dpp_f<0x138>(fill, x); }

__device__ __forceinline__ float readlane_f(float x, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

// min over the 64 lanes, returned wave-uniform
__device__ __forceinline__ float wave_min(float x) {
  const float inf = INFINITY;
  x = fminf(x, dpp_f<0x111>(inf, x));        // row_shr:1
  x = fminf(x, dpp_f<0x112>(inf, x));        // row_shr:2
  x = fminf(x, dpp_f<0x114>(inf, x));        // row_shr:4
  x = fminf(x, dpp_f<0x118>(inf, x));        // row_shr:8  -> lane 15 of each row holds the row min
  x = fminf(x, dpp_f<0x142, 0xa>(inf, x));   // row_bcast:15 into rows 1 and 3
  x = fminf(x, dpp_f<0x143, 0xc>(inf, x));   // row_bcast:31 into rows 2 and 3
  return readlane_f(x, 63);
}

// sum over the 64 lanes, returned wave-uniform
__device__ __forceinline__ float wave_sum(float x) {
  x += dpp_f<0x111>(0.f, x);
  x += dpp_f<0x112>(0.f, x);
  x += dpp_f<0x114>(0.f, x);
  x += dpp_f<0x118>(0.f, x);
  x += dpp_f<0x142, 0xa>(0.f, x);
  x += dpp_f<0x143, 0xc>(0.f, x);
  return readlane_f(x, 63);
}

__device__ __forceinline__ uint64_t ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }

// largest label (R*lane + j) whose predicate is set; `dflt` when none is
template <int R>
__device__ __forceinline__ int last_label(const bool (&pred)[R], int dflt) {
  uint64_t m[R];
  uint64_t any = 0;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    m[j] = ballot(pred[j]);
    any |= m[j];
  }
  if (any == 0) return dflt;
  int lane = 63 - __builtin_clzll(any);
  int jj = 0;
#pragma unroll
  for (int j = 0; j < R; ++j)
    if ((m[j] >> lane) & 1) jj = j;
  return R * lane + jj;
}

// ------------------------------------------------------------------------------------------------
// label-vector access: lane owns labels lab0 .. lab0+R-1
// ------------------------------------------------------------------------------------------------
template <int R>
struct __attribute__((packed, aligned(4))) VecF {
  float v[R];
};
template <int R>
struct __attribute__((packed, aligned(1))) VecB {
  uint8_t v[R];
};

struct Lane {
  int lab0;    // first label of this lane
  int nvalid;  // how many of its R labels exist (0..R)
};

template <int R>
__device__ __forceinline__ void load_vec(const float* __restrict__ base, const Lane ln,
                                         float (&x)[R], float fill) {
  if (ln.nvalid == R) {
    VecF<R> t = *reinterpret_cast<const VecF<R>*>(base + ln.lab0);
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = t.v[j];
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = (j < ln.nvalid) ? base[ln.lab0 + j] : fill;
  }
}

template <int R>
__device__ __forceinline__ void store_vec(float* __restrict__ base, const Lane ln,
                                          const float (&x)[R]) {
  if (ln.nvalid == R) {
    VecF<R> t;
#pragma unroll
    for (int j = 0; j < R; ++j) t.v[j] = x[j];
    *reinterpret_cast<VecF<R>*>(base + ln.lab0) = t;
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j)
      if (j < ln.nvalid) base[ln.lab0 + j] = x[j];
  }
}

template <int R>
__device__ __forceinline__ void load_idx(const uint8_t* __restrict__ base, const Lane ln,
                                         int (&x)[R]) {
  if (ln.nvalid == R) {
    VecB<R> t = *reinterpret_cast<const VecB<R>*>(base + ln.lab0);
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = t.v[j];
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = (j < ln.nvalid) ? base[ln.lab0 + j] : 0;
  }
}

template <int R>
__device__ __forceinline__ void store_idx(uint8_t* __restrict__ base, const Lane ln,
                                          const int (&x)[R]) {
  if (ln.nvalid == R) {
    VecB<R> t;
#pragma unroll
    for (int j = 0; j < R; ++j) t.v[j] = (uint8_t)x[j];
    *reinterpret_cast<VecB<R>*>(base + ln.lab0) = t;
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j)
      if (j < ln.nvalid) base[ln.lab0 + j] = (uint8_t)x[j];
  }
}

// ------------------------------------------------------------------------------------------------
// chain geometry.  Direction table: MPLayers/common.cpp:28-76.  A chain starts at every pixel whose
// front neighbour (pixel - step) lies outside the image; that reproduces the reference's trees
// (common.cpp:78-87 and the start formulas of the scan kernels) without empty chains.
// ------------------------------------------------------------------------------------------------
struct DirGeom {
  int hs, ws;   // step of the forward scan
  int ha, wa;   // |hs|, |ws| clipped to the image
  int count_a;  // chains starting in the first ha rows the scan enters
  int n_chains;
};

__host__ __device__ inline void dir_step(int dir, int* hs, int* ws) {
  const int tab[16][2] = {{0, 1},  {0, -1}, {1, 0},  {-1, 0},  {1, 1},  {-1, -1}, {1, -1}, {-1, 1},
                          {1, 2},  {-1, -2}, {2, 1}, {-2, -1}, {2, -1}, {-2, 1},  {1, -2}, {-1, 2}};
  *hs = tab[dir][0];
  *ws = tab[dir][1];
}

__host__ __device__ inline DirGeom make_dir(int dir, int H, int W) {
  DirGeom g;
  dir_step(dir, &g.hs, &g.ws);
  int ha = g.hs < 0 ? -g.hs : g.hs, wa = g.ws < 0 ? -g.ws : g.ws;
  g.ha = ha < H ? ha : H;
  g.wa = wa < W ? wa : W;
  g.count_a = g.ha * W;
  g.n_chains = g.count_a + (H - g.ha) * g.wa;
  return g;
}

// start pixel (h, w) and number of pixels n (>= 1) of chain c
__device__ __forceinline__ void chain_start(const DirGeom& g, int H, int W, int c, int* h, int* w,
                                            int* n) {
  int hh, ww;
  if (c < g.count_a) {
    int r = c / W;
    ww = c - r * W;
    hh = g.hs > 0 ? r : H - 1 - r;
  } else {
    int cc = c - g.count_a;
    int r = cc / g.wa;
    int k = cc - r * g.wa;
    hh = g.hs > 0 ? g.ha + r : (g.hs < 0 ? H - 1 - g.ha - r : r);
    ww = g.ws > 0 ? k : W - 1 - k;
  }
  int nh = 0x7fffffff, nw = 0x7fffffff;
  if (g.hs > 0) nh = (H - 1 - hh) / g.hs;
  if (g.hs < 0) nh = hh / (-g.hs);
  if (g.ws > 0) nw = (W - 1 - ww) / g.ws;
  if (g.ws < 0) nw = ww / (-g.ws);
  *h = hh;
  *w = ww;
  *n = 1 + (nh < nw ? nh : nw);
}

// ------------------------------------------------------------------------------------------------
// context descriptor, computed on the device so that no host round trip is needed
// ------------------------------------------------------------------------------------------------
struct CtxDesc {
  int band_k;     // > 0: c[k] == cmax for all k >= band_k and c[k] <= cmax below; 0: dense path
  int c0_is_min;  // c[0] <= c[k] for all k
  float cmax;
  int pad;
};

// 1-D context c[0..L-1]: find the constant tail.  One wave.
__global__ void __launch_bounds__(kWave) analyze_context_kernel(const float* __restrict__ ctx, int L,
                                                                int ctx2d, CtxDesc* __restrict__ d) {
  if (threadIdx.x != 0) return;
  CtxDesc r;
  r.band_k = 0;
  r.c0_is_min = 0;
  r.cmax = 0.f;
  r.pad = 0;
  if (!ctx2d) {
    float tail = ctx[L - 1];
    int k = L - 1;
    while (k > 0 && ctx[k - 1] == tail) --k;  // c[k..L-1] == tail
    bool ok = (tail == tail);
    bool c0min = true;
    for (int i = 0; i < L; ++i) {
      float v = ctx[i];
      if (!(v <= tail)) ok = false;
      if (!(ctx[0] <= v)) c0min = false;
    }
    if (k < 1) k = 1;  // a constant context: the centre tap alone is the band
    if (ok && k <= kMaxBandK) {
      r.band_k = k;
      r.cmax = tail;
      r.c0_is_min = c0min ? 1 : 0;
    }
  }
  *d = r;
}

// ------------------------------------------------------------------------------------------------
// forward sweep
// ------------------------------------------------------------------------------------------------
struct SweepParams {
  int B, H, W, L;
  int ctx2d;
  int n_dirs;                        // directions in this launch
  int dirs[kMaxDirs];                // their ids
  int block_prefix[kMaxDirs + 1];    // prefix sums of B * n_chains
  float rho;
  const float* belief;               // S plane (N)
  float* belief_out;                 // TRWP: == belief; Jacobi: unused
  const float* msg_in;               // (n_dir_total, N) planes read
  float* msg_out;                    // (n_dir_total, N) planes written
  const float* edge;                 // (n_dir_total, P)
  const float* ctx;
  const CtxDesc* desc;               // may be null: dense path
  uint8_t* idx_min;                  // (n_dir_total, N) of this iteration, or null
  uint8_t* idx_norm;                 // (n_dir_total, P) of this iteration, or null
};

template <int R>
struct PixF {
  float s[R], md[R], mi[R];
  float w;
};

struct ChainCtx {
  int64_t pix0;   // linear pixel index of the chain start
  int64_t pstep;  // pixel stride along the chain
  int n;          // pixels in the chain
};

template <int R>
__device__ __forceinline__ PixF<R> load_pix_fwd(const float* __restrict__ S,
                                                const float* __restrict__ md,
                                                const float* __restrict__ mi,
                                                const float* __restrict__ w, const ChainCtx& ch,
                                                int t, int L, const Lane ln) {
  PixF<R> r;
  t = t < ch.n ? t : ch.n - 1;
  int64_t pix = ch.pix0 + (int64_t)t * ch.pstep;
  int64_t off = pix * L;
  if (ln.nvalid > 0) {
    load_vec<R>(S + off, ln, r.s, 0.f);
    load_vec<R>(md + off, ln, r.md, 0.f);
    load_vec<R>(mi + off, ln, r.mi, 0.f);
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j) r.s[j] = r.md[j] = r.mi[j] = 0.f;
  }
  r.w = w[pix];
  return r;
}

// Dense O(L^2) step: v[cd] = min_fd( a[fd] + w * ctx(cd, fd) ), largest fd on ties.
// HorizontalKernel inner loop, TRWP_forward.cu:127-153.  a_s / ctx_s live in LDS.
template <int R, bool TRAIN>
__device__ __forceinline__ void dense_step(const float (&a)[R], float w, int L, int ctx2d,
                                           const Lane ln, float* a_s, const float* ctx_s,
                                           float (&v)[R], int (&fd_idx)[R]) {
#pragma unroll
  for (int j = 0; j < R; ++j)
    if (j < ln.nvalid) a_s[ln.lab0 + j] = a[j];
  __syncthreads();
  int labc[R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    int l = ln.lab0 + j;
    labc[j] = l < L ? l : L - 1;
    v[j] = INFINITY;
    fd_idx[j] = L - 1;
  }
  for (int fd = L - 1; fd >= 0; --fd) {
    float af = a_s[fd];
#pragma unroll
    for (int j = 0; j < R; ++j) {
      int cd = labc[j];
      int ci = ctx2d ? (cd < fd ? cd * L + fd : fd * L + cd) : (cd > fd ? cd - fd : fd - cd);
      float val = fmaf(w, ctx_s[ci], af);
      bool take = (fd == L - 1) || (val < v[j]);
      v[j] = take ? val : v[j];
      if (TRAIN) fd_idx[j] = take ? fd : fd_idx[j];
    }
  }
  __syncthreads();
}

// Band O(L*K) step for 1-D contexts with a constant tail: exact for w >= 0 (see CtxDesc).
//   v[cd] = min( min_{|k|<K} a[cd+k] + w*c[|k|],  min_fd a[fd] + w*cmax )
// KT > 0: K known at compile time, taps c[] in registers.  KT == 0: K at run time, taps in LDS.
template <int R, bool TRAIN, int KT>
__device__ __forceinline__ void band_step(const float (&a)[R], float w, int K, const float* c_reg,
                                          const float* ctx_s, float cmax, float amin, int fstar,
                                          const Lane ln, float (&v)[R], int (&fd_idx)[R]) {
  const float inf = INFINITY;
  float up[R], dn[R];
  int off[R];
  const float c0 = KT > 0 ? c_reg[0] : ctx_s[0];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    up[j] = a[j];
    dn[j] = a[j];
    v[j] = fmaf(w, c0, a[j]);
    off[j] = 0;
  }
  auto tap = [&](int k, float ck) {
    // one-label shifts: up[j] <- a[label + k], dn[j] <- a[label - k]
    float tu = wave_shl1(up[0], inf);
    float td = wave_shr1(dn[R - 1], inf);
#pragma unroll
    for (int j = 0; j < R - 1; ++j) up[j] = up[j + 1];
    up[R - 1] = tu;
#pragma unroll
    for (int j = R - 1; j > 0; --j) dn[j] = dn[j - 1];
    dn[0] = td;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      float cu = fmaf(w, ck, up[j]);
      float cd = fmaf(w, ck, dn[j]);
      if (TRAIN) {
        bool tk = cu <= v[j];  // larger front label wins ties
        v[j] = tk ? cu : v[j];
        off[j] = tk ? k : off[j];
        bool tk2 = cd < v[j];  // smaller front label loses ties
        v[j] = tk2 ? cd : v[j];
        off[j] = tk2 ? -k : off[j];
      } else {
        v[j] = fminf(v[j], fminf(cu, cd));
      }
    }
  };
  if (KT > 0) {
#pragma unroll
    for (int k = 1; k < KT; ++k) tap(k, c_reg[k]);
  } else {
    for (int k = 1; k < K; ++k) tap(k, ctx_s[k]);
  }
  const float far = fmaf(w, cmax, amin);
#pragma unroll
  for (int j = 0; j < R; ++j) {
    if (TRAIN) {
      int fb = ln.lab0 + j + off[j];
      bool lt = far < v[j];
      bool eq = far == v[j];
      int fe = fb > fstar ? fb : fstar;
      fd_idx[j] = lt ? fstar : (eq ? fe : fb);
      v[j] = lt ? far : v[j];
    } else {
      v[j] = fminf(v[j], far);
    }
  }
}

// One chain.  KT: > 0 band with compile-time K, 0 band with run-time K, -1 dense.
template <int R, bool TRAIN, bool JACOBI, int KT>
__device__ __forceinline__ void run_chain_fwd(const SweepParams& p, const CtxDesc& desc, int dir,
                                              const ChainCtx& ch, const Lane ln, float* a_s,
                                              const float* ctx_s) {
  const int L = p.L;
  const int64_t N = (int64_t)p.B * p.H * p.W * L;
  const int64_t P = (int64_t)p.B * p.H * p.W;
  const float* __restrict__ S = p.belief;
  const float* __restrict__ md = p.msg_in + (int64_t)dir * N;
  const float* __restrict__ mi = p.msg_in + (int64_t)(dir ^ 1) * N;
  const float* __restrict__ wp = p.edge + (int64_t)dir * P;
  float* __restrict__ mo = p.msg_out + (int64_t)dir * N;
  float* __restrict__ So = p.belief_out;
  uint8_t* __restrict__ imin = TRAIN ? p.idx_min + (int64_t)dir * N : nullptr;
  uint8_t* __restrict__ inorm = TRAIN ? p.idx_norm + (int64_t)dir * P : nullptr;
  const float rho = p.rho;
  const float inf = INFINITY;
  const int lane = threadIdx.x;

  float c_reg[KT > 0 ? KT : 1];
  if (KT > 0) {
#pragma unroll
    for (int k = 0; k < KT; ++k) c_reg[k] = p.ctx[k];
  }
  const int K = desc.band_k;
  const float cmax = desc.cmax;
  const bool c0min = desc.c0_is_min != 0;

  PixF<R> ring[kPrefetch];
#pragma unroll
  for (int u = 0; u < kPrefetch; ++u) ring[u] = load_pix_fwd<R>(S, md, mi, wp, ch, u, L, ln);

  float prev[R], uf[R];
#pragma unroll
  for (int j = 0; j < R; ++j) prev[j] = uf[j] = 0.f;

  for (int t0 = 0; t0 < ch.n; t0 += kPrefetch) {
#pragma unroll
    for (int u = 0; u < kPrefetch; ++u) {
      const int t = t0 + u;
      if (t >= ch.n) break;
      const PixF<R> px = ring[u];
      ring[u] = load_pix_fwd<R>(S, md, mi, wp, ch, t + kPrefetch, L, ln);
      const int64_t pix = ch.pix0 + (int64_t)t * ch.pstep;
      float tt[R], un[R];
#pragma unroll
      for (int j = 0; j < R; ++j) {
        tt[j] = px.s[j] - px.md[j];             // unary + sum of the other directions' messages
        un[j] = fmaf(tt[j], rho, -px.mi[j]);    // UpdateUnaryKernel, TRWP_forward.cu:70-78
      }
      if (t == 0) {
        // chain start: its front lies outside the image, the reference never writes it.
        // Jacobi buffers alternate, so the start pixel is written with the zeros it keeps there.
        if (JACOBI && ln.nvalid > 0) {
          float z[R];
#pragma unroll
          for (int j = 0; j < R; ++j) z[j] = 0.f;
          store_vec<R>(mo + pix * L, ln, z);
        }
      } else {
        const float w = __builtin_bit_cast(
            float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, px.w)));
        float a[R], v[R];
        int fd_idx[R];
#pragma unroll
        for (int j = 0; j < R; ++j) a[j] = (j < ln.nvalid) ? fmaf(rho, prev[j], uf[j]) : inf;
        float nmin;
        bool need_nmin = true;
        if (KT >= 0 && w >= 0.f) {
          float am = a[0];
#pragma unroll
          for (int j = 1; j < R; ++j) am = fminf(am, a[j]);
          const float amin = wave_min(am);
          int fstar = L - 1;
          if (TRAIN) {
            bool pr[R];
#pragma unroll
            for (int j = 0; j < R; ++j) pr[j] = (a[j] == amin);
            fstar = last_label<R>(pr, L - 1);
          }
          band_step<R, TRAIN, (KT > 0 ? KT : 0)>(a, w, K, c_reg, ctx_s, cmax, amin, fstar, ln, v,
                                                 fd_idx);
          if (c0min) {
            // every candidate is >= amin + w*c[0], which the centre tap of label argmin(a) attains
            nmin = fmaf(w, KT > 0 ? c_reg[0] : ctx_s[0], amin);
            need_nmin = false;
          }
        } else {
          dense_step<R, TRAIN>(a, w, L, p.ctx2d, ln, a_s, ctx_s, v, fd_idx);
        }
        if (need_nmin) {
          float vm = inf;
#pragma unroll
          for (int j = 0; j < R; ++j) vm = fminf(vm, (j < ln.nvalid) ? v[j] : inf);
          nmin = wave_min(vm);
        }
        float m[R], sn[R];
#pragma unroll
        for (int j = 0; j < R; ++j) {
          m[j] = v[j] - nmin;  // MsgNormNaive, commonCUDA.cuh:126-128
          sn[j] = tt[j] + m[j];
        }
        if (ln.nvalid > 0) {
          store_vec<R>(mo + pix * L, ln, m);
          if (!JACOBI) store_vec<R>(So + pix * L, ln, sn);
          if (TRAIN) store_idx<R>(imin + pix * L, ln, fd_idx);
        }
        if (TRAIN) {
          bool pr[R];
#pragma unroll
          for (int j = 0; j < R; ++j) pr[j] = (j < ln.nvalid) && (v[j] == nmin);
          int nidx = last_label<R>(pr, L - 1);
          if (lane == 0) inorm[pix] = (uint8_t)nidx;
        }
#pragma unroll
        for (int j = 0; j < R; ++j) prev[j] = m[j];
      }
#pragma unroll
      for (int j = 0; j < R; ++j) uf[j] = un[j];
    }
  }
}

template <int R, bool TRAIN, bool JACOBI>
__global__ void __launch_bounds__(kWave) sweep_fwd_kernel(const SweepParams p) {
  extern __shared__ float smem[];
  float* a_s = smem;             // kMaxL floats
  float* ctx_s = smem + kMaxL;   // L or L*L floats
  const int lane = threadIdx.x;
  const int L = p.L;

  // which direction / chain does this wave own
  int di = 0;
  while (di + 1 < p.n_dirs && (int)blockIdx.x >= p.block_prefix[di + 1]) ++di;
  const int dir = p.dirs[di];
  const int local = (int)blockIdx.x - p.block_prefix[di];
  const DirGeom g = make_dir(dir, p.H, p.W);
  const int bv = local / g.n_chains;
  const int c = local - bv * g.n_chains;
  int h0, w0, n;
  chain_start(g, p.H, p.W, c, &h0, &w0, &n);
  ChainCtx ch;
  ch.pix0 = ((int64_t)bv * p.H + h0) * p.W + w0;
  ch.pstep = (int64_t)g.hs * p.W + g.ws;
  ch.n = n;
  if (!JACOBI && n < 2) return;  // nothing to write

  Lane ln;
  ln.lab0 = R * lane;
  int nv = L - ln.lab0;
  ln.nvalid = nv < 0 ? 0 : (nv > R ? R : nv);

  CtxDesc desc;
  if (p.desc != nullptr) {
    desc = *p.desc;
  } else {
    desc.band_k = 0;
    desc.c0_is_min = 0;
    desc.cmax = 0.f;
    desc.pad = 0;
  }
  // context table into LDS (dense path, run-time band taps, negative-weight fallback)
  const int n_ctx = p.ctx2d ? L * L : L;
  for (int i = lane; i < n_ctx; i += kWave) ctx_s[i] = p.ctx[i];
  __syncthreads();

  switch (desc.band_k) {
    case 0: run_chain_fwd<R, TRAIN, JACOBI, -1>(p, desc, dir, ch, ln, a_s, ctx_s); break;
    case 1: run_chain_fwd<R, TRAIN, JACOBI, 1>(p, desc, dir, ch, ln, a_s, ctx_s); break;
    case 2: run_chain_fwd<R, TRAIN, JACOBI, 2>(p, desc, dir, ch, ln, a_s, ctx_s); break;
    case 3: run_chain_fwd<R, TRAIN, JACOBI, 3>(p, desc, dir, ch, ln, a_s, ctx_s); break;
    case 4: run_chain_fwd<R, TRAIN, JACOBI, 4>(p, desc, dir, ch, ln, a_s, ctx_s); break;
    case 5: run_chain_fwd<R, TRAIN, JACOBI, 5>(p, desc, dir, ch, ln, a_s, ctx_s); break;
    default: run_chain_fwd<R, TRAIN, JACOBI, 0>(p, desc, dir, ch, ln, a_s, ctx_s); break;
  }
}

// ------------------------------------------------------------------------------------------------
// elementwise kernels
// ------------------------------------------------------------------------------------------------
// S = unary + sum_k m_k  (k ascending, as UpdateUnaryKernel sums, TRWP_forward.cu:70-73)
__global__ void __launch_bounds__(256) belief_kernel(const float* __restrict__ unary,
                                                     const float* __restrict__ msg, int n_dir,
                                                     int64_t N, float* __restrict__ S) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N;
       i += (int64_t)gridDim.x * blockDim.x) {
    float v = unary[i];
    for (int k = 0; k < n_dir; ++k) v += msg[(int64_t)k * N + i];
    S[i] = v;
  }
}

// cost = factor*unary + sum_k m_k  (or + min_k m_k): CostAggregateKernel, TRWP_forward.cu:31-58,
// ISGMR_forward.cu:69-99.  copy_to != null: also mirror the message planes there.
__global__ void __launch_bounds__(256) aggregate_kernel(const float* __restrict__ unary,
                                                        const float* __restrict__ msg, int n_dir,
                                                        int64_t N, float factor, int min_a_dir,
                                                        float* __restrict__ cost,
                                                        float* __restrict__ copy_to) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N;
       i += (int64_t)gridDim.x * blockDim.x) {
    float v = unary[i] * factor;
    if (min_a_dir) {
      float mn = msg[i];
      if (copy_to) copy_to[i] = mn;
      for (int k = 1; k < n_dir; ++k) {
        float m = msg[(int64_t)k * N + i];
        if (copy_to) copy_to[(int64_t)k * N + i] = m;
        if (m < mn) mn = m;
      }
      v += mn;
    } else {
      for (int k = 0; k < n_dir; ++k) {
        float m = msg[(int64_t)k * N + i];
        if (copy_to) copy_to[(int64_t)k * N + i] = m;
        v += m;
      }
    }
    cost[i] = v;
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

// ------------------------------------------------------------------------------------------------
// backward sweep
// ------------------------------------------------------------------------------------------------
struct BackParams {
  int B, H, W, L;
  int ctx2d;
  int jacobi;
  int n_dirs;
  int dirs[kMaxDirs];
  int block_prefix[kMaxDirs + 1];
  float rho;
  // TRWP: g_k = A + h_k.  a_in: plane read as A (dcost_final on the first sweep), a_out: dunary.
  const float* a_in;
  float* a_out;
  float* h;                 // (n_dir_total, N) planes h_k
  int first_touch;          // h_dir and h_inv have not been written yet: read as zero
  // ISGMR: gu_in planes (plane stride gu_stride; 0 on the first iteration where gu_k = dcost_final),
  // du_out (n_dir_total, N) receives dU_d in place of gu_d
  const float* gu_in;
  int64_t gu_stride;
  float* du_out;
  const float* edge;        // (n_dir_total, P)
  const float* ctx;
  const uint8_t* idx_min;   // (n_dir_total, N) of this iteration
  const uint8_t* idx_norm;  // (n_dir_total, P)
  float* dedge;             // (n_dir_total, P) accumulates
  float* dctx;              // accumulates
};

template <int R>
struct PixB {
  float a[R], hd[R], hi[R];
  int fd[R];
  int nidx;
  float w;
};

template <int R, bool JACOBI>
__device__ __forceinline__ PixB<R> load_pix_bwd(const BackParams& p, const float* __restrict__ A,
                                                const float* __restrict__ hd,
                                                const float* __restrict__ hi,
                                                const uint8_t* __restrict__ imin,
                                                const uint8_t* __restrict__ inorm,
                                                const float* __restrict__ w, const ChainCtx& ch,
                                                int t, int L, const Lane ln) {
  PixB<R> r;
  t = t > 0 ? t : 0;
  int64_t pix = ch.pix0 + (int64_t)t * ch.pstep;
  int64_t off = pix * L;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    r.a[j] = r.hd[j] = r.hi[j] = 0.f;
    r.fd[j] = 0;
  }
  if (ln.nvalid > 0) {
    load_vec<R>(A + off, ln, r.a, 0.f);
    if (!JACOBI && !p.first_touch) {
      load_vec<R>(hd + off, ln, r.hd, 0.f);
      load_vec<R>(hi + off, ln, r.hi, 0.f);
    }
    load_idx<R>(imin + off, ln, r.fd);
  }
  r.nidx = inorm[pix];
  r.w = w[pix];
  return r;
}

// Reverse scan of one chain: HorizontalKernelBack & co, TRWP_backward.cu:49-275, fused with
// UpdateUnaryKernelBack (:26-47) and the two memsets (:421-422).
template <int R, bool JACOBI>
__global__ void __launch_bounds__(kWave) sweep_bwd_kernel(const BackParams p) {
  extern __shared__ float smem[];
  float* sc_s = smem;                                        // kMaxL floats
  float* ctx_s = smem + kMaxL;                               // L or L*L floats
  float* hist_s = ctx_s + (p.ctx2d ? p.L * p.L : p.L);       // same size
  const int lane = threadIdx.x;
  const int L = p.L;
  const int64_t P = (int64_t)p.B * p.H * p.W;
  const int64_t N = P * L;

  int di = 0;
  while (di + 1 < p.n_dirs && (int)blockIdx.x >= p.block_prefix[di + 1]) ++di;
  const int dir = p.dirs[di];
  const int local = (int)blockIdx.x - p.block_prefix[di];
  const DirGeom g = make_dir(dir, p.H, p.W);
  const int bv = local / g.n_chains;
  const int c = local - bv * g.n_chains;
  int h0, w0, n;
  chain_start(g, p.H, p.W, c, &h0, &w0, &n);
  ChainCtx ch;
  ch.pix0 = ((int64_t)bv * p.H + h0) * p.W + w0;
  ch.pstep = (int64_t)g.hs * p.W + g.ws;
  ch.n = n;

  Lane ln;
  ln.lab0 = R * lane;
  int nv = L - ln.lab0;
  ln.nvalid = nv < 0 ? 0 : (nv > R ? R : nv);

  const int n_ctx = p.ctx2d ? L * L : L;
  for (int i = lane; i < n_ctx; i += kWave) {
    ctx_s[i] = p.ctx[i];
    hist_s[i] = 0.f;
  }
  __syncthreads();

  const float* __restrict__ A = JACOBI ? p.gu_in + (int64_t)dir * p.gu_stride : p.a_in;
  float* __restrict__ Ao = JACOBI ? p.du_out + (int64_t)dir * N : p.a_out;
  float* __restrict__ hd = JACOBI ? nullptr : p.h + (int64_t)dir * N;
  float* __restrict__ hi = JACOBI ? nullptr : p.h + (int64_t)(dir ^ 1) * N;
  const uint8_t* __restrict__ imin = p.idx_min + (int64_t)dir * N;
  const uint8_t* __restrict__ inorm = p.idx_norm + (int64_t)dir * P;
  const float* __restrict__ wp = p.edge + (int64_t)dir * P;
  float* __restrict__ dedge = p.dedge + (int64_t)dir * P;
  const float rho = p.rho;

  PixB<R> ring[kPrefetch];
#pragma unroll
  for (int u = 0; u < kPrefetch; ++u)
    ring[u] = load_pix_bwd<R, JACOBI>(p, A, hd, hi, imin, inorm, wp, ch, n - 1 - u, L, ln);

  float sc[R];  // dU of the current pixel: what the previous step scattered into it
#pragma unroll
  for (int j = 0; j < R; ++j) sc[j] = 0.f;

  for (int s0 = 0; s0 < n; s0 += kPrefetch) {
#pragma unroll
    for (int u = 0; u < kPrefetch; ++u) {
      const int s = s0 + u;
      if (s >= n) break;
      const int t = n - 1 - s;
      const PixB<R> px = ring[u];
      ring[u] = load_pix_bwd<R, JACOBI>(p, A, hd, hi, imin, inorm, wp, ch, t - kPrefetch, L, ln);
      const int64_t pix = ch.pix0 + (int64_t)t * ch.pstep;
      float scn[R];
#pragma unroll
      for (int j = 0; j < R; ++j) scn[j] = 0.f;
      if (t >= 1) {
        const float w = __builtin_bit_cast(
            float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, px.w)));
        const int nidx = __builtin_amdgcn_readfirstlane(px.nidx);
        float gv[R];
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
          // gradient w.r.t. the normalised message of this pixel, including what the previous
          // step added through the recurrence (dmsg[front] += rho * value, TRWP_backward.cu:108)
          float base = JACOBI ? px.a[j] : (px.a[j] + px.hd[j]);
          gv[j] = (j < ln.nvalid) ? fmaf(rho, sc[j], base) : 0.f;
          part += gv[j];
        }
        const float tot = wave_sum(part);  // MsgNormNaiveBack, commonCUDA.cuh:131-145
        float de = 0.f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
          if (ln.lab0 + j == nidx) gv[j] -= tot;
          if (j < ln.nvalid) sc_s[ln.lab0 + j] = 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; ++j) {
          if (j < ln.nvalid) {
            const int cd = ln.lab0 + j, fd = px.fd[j];
            const int ci = p.ctx2d ? (cd < fd ? cd * L + fd : fd * L + cd)
                                   : (cd > fd ? cd - fd : fd - cd);
            atomicAdd(&sc_s[fd], gv[j]);                       // dunary_update[front, fd] += value
            de = fmaf(ctx_s[ci], gv[j], de);                   // dedge_weights[cur] += ctx * value
            if (cd != fd) atomicAdd(&hist_s[ci], w * gv[j]);   // dcontext += edge_weight * value
          }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; ++j) scn[j] = (j < ln.nvalid) ? sc_s[ln.lab0 + j] : 0.f;
        const float det = wave_sum(de);
        if (lane == 0) atomicAdd(&dedge[pix], det);
      }
      // pixel-local part of UpdateUnaryKernelBack with dU[pix] = sc
      if (ln.nvalid > 0) {
        if (JACOBI) {
          store_vec<R>(Ao + pix * L, ln, sc);
        } else {
          float an[R], hdn[R], hin[R];
#pragma unroll
          for (int j = 0; j < R; ++j) {
            an[j] = fmaf(rho, sc[j], px.a[j]);  // g_k += rho*dU for every k, dunary too
            hdn[j] = -an[j];                    // g_dir = 0 after its sweep
            hin[j] = px.hi[j] - sc[j];          // g_inv -= dU
          }
          store_vec<R>(Ao + pix * L, ln, an);
          store_vec<R>(hd + pix * L, ln, hdn);
          store_vec<R>(hi + pix * L, ln, hin);
        }
      }
#pragma unroll
      for (int j = 0; j < R; ++j) sc[j] = scn[j];
    }
  }
  __syncthreads();
  for (int i = lane; i < n_ctx; i += kWave) {
    float v = hist_s[i];
    if (v != 0.f) atomicAdd(&p.dctx[i], v);
  }
}

// ISGMR: after all directions of an iteration have been scanned back (X_k = dU_k):
//   dunary += rho * sum_k X_k ;  gu_k = rho * (sum - X_k) - X_{k^1}
// (UpdateUnaryKernelBack summed over directions + SumMsgKernel, ISGMR_backward.cu:39-60, 482-483)
__global__ void __launch_bounds__(256) isgmr_combine_kernel(float* __restrict__ X, int n_dir,
                                                            int64_t N, float rho,
                                                            const float* __restrict__ dcost,
                                                            float factor, int init_dunary,
                                                            int write_gu,
                                                            float* __restrict__ dunary) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N;
       i += (int64_t)gridDim.x * blockDim.x) {
    float x[kMaxDirs];
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < kMaxDirs; ++k) {
      x[k] = (k < n_dir) ? X[(int64_t)k * N + i] : 0.f;
    }
    for (int k = n_dir - 1; k >= 0; --k) sum += x[k];
    float du = init_dunary ? factor * dcost[i] : dunary[i];
    dunary[i] = fmaf(rho, sum, du);
    if (write_gu) {
#pragma unroll
      for (int k = 0; k < kMaxDirs; ++k)
        if (k < n_dir) X[(int64_t)k * N + i] = fmaf(rho, sum - x[k], -x[k ^ 1]);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// wave-primitive self test
// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kWave) selftest_kernel(int* out) {
  const int lane = threadIdx.x;
  int ok = 1;
  float x = (float)(lane * 3 % 17) + 100.f;
  float up = wave_shl1(x, -1.f);
  float dn = wave_shr1(x, -2.f);
  float eu = lane < 63 ? (float)((lane + 1) * 3 % 17) + 100.f : -1.f;
  float ed = lane > 0 ? (float)((lane - 1) * 3 % 17) + 100.f : -2.f;
  if (up != eu || dn != ed) ok = 0;
  float y = (float)((lane * 37 + 11) % 64);  // a permutation of 0..63
  if (wave_min(y) != 0.f) ok = 0;
  for (int special = 0; special < 64; special += 9)  // the minimum sits in every row and bank
    if (wave_min(y + (lane == special ? -100.f : 0.f)) != (float)((special * 37 + 11) % 64) - 100.f)
      ok = 0;
  if (wave_sum((float)lane) != 2016.f) ok = 0;
  bool pr[2] = {lane == 5 || lane == 40, lane == 40};
  if (last_label<2>(pr, -1) != 81) ok = 0;
  bool pn[2] = {false, false};
  if (last_label<2>(pn, -7) != -7) ok = 0;
  uint64_t b = ballot(ok != 0);
  if (lane == 0) {
    out[0] = (b == ~0ull) ? 1 : 0;
    out[1] = (int)(b & 0xffffffffu);
    out[2] = (int)(b >> 32);
  }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

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

int elementwise_blocks(int64_t n) {
  int64_t b = (n + 256 * 4 - 1) / (256 * 4);
  if (b < 1) b = 1;
  if (b > 256 * 32) b = 256 * 32;
  return (int)b;
}

void fill_dirs(const mpl_shape* s, int first, int count, int* dirs, int* prefix, int* n_dirs) {
  *n_dirs = count;
  prefix[0] = 0;
  for (int i = 0; i < count; ++i) {
    dirs[i] = first + i;
    prefix[i + 1] = prefix[i] + s->batch * make_dir(first + i, s->height, s->width).n_chains;
  }
}

template <bool TRAIN, bool JACOBI>
void launch_fwd(const SweepParams& p, hipStream_t st) {
  const int R = (p.L + kWave - 1) / kWave;
  const int blocks = p.block_prefix[p.n_dirs];
  if (blocks <= 0) return;
  const size_t lds = sizeof(float) * (kMaxL + (p.ctx2d ? p.L * p.L : p.L));
  switch (R) {
    case 1: sweep_fwd_kernel<1, TRAIN, JACOBI><<<blocks, kWave, lds, st>>>(p); break;
    case 2: sweep_fwd_kernel<2, TRAIN, JACOBI><<<blocks, kWave, lds, st>>>(p); break;
    case 3: sweep_fwd_kernel<3, TRAIN, JACOBI><<<blocks, kWave, lds, st>>>(p); break;
    default: sweep_fwd_kernel<4, TRAIN, JACOBI><<<blocks, kWave, lds, st>>>(p); break;
  }
}

template <bool JACOBI>
void launch_bwd(const BackParams& p, hipStream_t st) {
  const int R = (p.L + kWave - 1) / kWave;
  const int blocks = p.block_prefix[p.n_dirs];
  if (blocks <= 0) return;
  const size_t lds = sizeof(float) * (kMaxL + 2 * (p.ctx2d ? p.L * p.L : p.L));
  switch (R) {
    case 1: sweep_bwd_kernel<1, JACOBI><<<blocks, kWave, lds, st>>>(p); break;
    case 2: sweep_bwd_kernel<2, JACOBI><<<blocks, kWave, lds, st>>>(p); break;
    case 3: sweep_bwd_kernel<3, JACOBI><<<blocks, kWave, lds, st>>>(p); break;
    default: sweep_bwd_kernel<4, JACOBI><<<blocks, kWave, lds, st>>>(p); break;
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
  return p;
}

// cost_final is not written before the final aggregation, so its first bytes carry the context
// descriptor during the sweeps (no allocation, no state shared between streams).
const CtxDesc* make_desc(const mpl_shape* s, const float* ctx, float* cost_final, hipStream_t st) {
  int64_t N = (int64_t)s->batch * s->height * s->width * s->n_disp;
  if (N * (int64_t)sizeof(float) < (int64_t)sizeof(CtxDesc)) return nullptr;  // dense path
  CtxDesc* d = reinterpret_cast<CtxDesc*>(cost_final);
  analyze_context_kernel<<<1, kWave, 0, st>>>(ctx, s->n_disp, s->ctx2d ? 1 : 0, d);
  return d;
}

}  // namespace

// ------------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------------
extern "C" {

const char* mpl_last_error(void) { return g_err; }

int mpl_version(void) { return 100; }

int mpl_n_chains(int dir, int height, int width) {
  if (dir < 0 || dir >= kMaxDirs || height < 1 || width < 1) return -1;
  return make_dir(dir, height, width).n_chains;
}

int mpl_selftest_wave_ops(int* out_host) {
  if (out_host == nullptr) return fail(MPL_EINVAL, "out_host is null");
  int* d = nullptr;
  if (hipMalloc(&d, 8 * sizeof(int)) != hipSuccess) return fail(MPL_ELAUNCH, "hipMalloc failed");
  (void)hipMemset(d, 0, 8 * sizeof(int));
  selftest_kernel<<<1, kWave>>>(d);
  hipError_t e = hipDeviceSynchronize();
  if (e == hipSuccess) e = hipMemcpy(out_host, d, 8 * sizeof(int), hipMemcpyDeviceToHost);
  (void)hipFree(d);
  if (e != hipSuccess) return fail(MPL_ELAUNCH, "selftest: %s", hipGetErrorString(e));
  return MPL_OK;
}

int mpl_trwp_forward(const mpl_shape* s, float rho, int n_iter, int enable_min_a_dir,
                     const float* unary, const float* context, const float* edge_weights,
                     float* msg, float* cost_final, uint8_t* msg_min_index,
                     uint8_t* msg_norm_index, float* unary_update, uint8_t* label_all,
                     void* stream) {
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  if (!unary || !context || !edge_weights || !msg || !cost_final || !unary_update)
    return fail(MPL_EINVAL, "trwp_forward: null tensor pointer");
  if ((msg_min_index == nullptr) != (msg_norm_index == nullptr))
    return fail(MPL_EINVAL, "trwp_forward: msg_min_index and msg_norm_index go together");
  hipStream_t st = (hipStream_t)stream;
  const int64_t P = (int64_t)s->batch * s->height * s->width;
  const int64_t N = P * s->n_disp;
  const bool train = msg_min_index != nullptr;

  const CtxDesc* desc = make_desc(s, context, cost_final, st);
  belief_kernel<<<elementwise_blocks(N), 256, 0, st>>>(unary, msg, s->n_dir, N, unary_update);

  SweepParams p = base_fwd_params(s, rho, edge_weights, context, desc);
  p.belief = unary_update;
  p.belief_out = unary_update;
  p.msg_in = msg;
  p.msg_out = msg;
  for (int it = 0; it < n_iter; ++it) {
    for (int d = 0; d < s->n_dir; ++d) {  // Gauss-Seidel over directions: TRWP_forward.cu:440-518
      fill_dirs(s, d, 1, p.dirs, p.block_prefix, &p.n_dirs);
      if (train) {
        p.idx_min = msg_min_index + (int64_t)it * s->n_dir * N;
        p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
        launch_fwd<true, false>(p, st);
      } else {
        launch_fwd<false, false>(p, st);
      }
    }
    if (label_all) {
      int64_t waves = (P < 256 * 64) ? P : 256 * 64;
      label_kernel<<<(int)((waves + 3) / 4), 256, 0, st>>>(unary, msg, s->n_dir, P, s->n_disp, 1.f,
                                                           enable_min_a_dir, label_all + it * P);
    }
  }
  aggregate_kernel<<<elementwise_blocks(N), 256, 0, st>>>(unary, msg, s->n_dir, N, 1.f,
                                                          enable_min_a_dir, cost_final, nullptr);
  return launch_ok("trwp_forward");
}

int mpl_isgmr_forward(const mpl_shape* s, int enable_sgm, float rho, int n_iter,
                      int enable_min_a_dir, const float* unary, const float* context,
                      const float* edge_weights, float* msg, float* cost_final,
                      uint8_t* msg_min_index, uint8_t* msg_norm_index, float* unary_update,
                      float* msg_update, uint8_t* label_all, void* stream) {
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
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
  float* buf[2] = {msg, msg_update};
  for (int it = 0; it < n_iter; ++it) {
    // Jacobi over directions (ISGMR_forward.cu:506-622): every direction reads the old messages;
    // the two buffers alternate instead of being copied.
    const float* cur = buf[it & 1];
    float* nxt = buf[(it + 1) & 1];
    belief_kernel<<<elementwise_blocks(N), 256, 0, st>>>(unary, cur, s->n_dir, N, unary_update);
    p.msg_in = cur;
    p.msg_out = nxt;
    if (train) {
      p.idx_min = msg_min_index + (int64_t)it * s->n_dir * N;
      p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
      launch_fwd<true, true>(p, st);
    } else {
      launch_fwd<false, true>(p, st);
    }
    if (label_all) {
      int64_t waves = (P < 256 * 64) ? P : 256 * 64;
      label_kernel<<<(int)((waves + 3) / 4), 256, 0, st>>>(unary, nxt, s->n_dir, P, s->n_disp,
                                                           factor, enable_min_a_dir,
                                                           label_all + it * P);
    }
  }
  const float* fin = buf[n_iter & 1];
  aggregate_kernel<<<elementwise_blocks(N), 256, 0, st>>>(unary, fin, s->n_dir, N, factor,
                                                          enable_min_a_dir, cost_final,
                                                          (n_iter & 1) ? msg : nullptr);
  return launch_ok("isgmr_forward");
}

int mpl_trwp_backward(const mpl_shape* s, float rho, int n_iter, const float* context,
                      const float* edge_weights, const float* dcost_final,
                      const uint8_t* msg_min_index, const uint8_t* msg_norm_index, float* dunary,
                      float* dcontext, float* dedge_weights, float* dmsg, float* dunary_update,
                      void* stream) {
  (void)dunary_update;
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  if (!context || !edge_weights || !dcost_final || !msg_min_index || !msg_norm_index || !dunary ||
      !dcontext || !dedge_weights || !dmsg)
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
  p.jacobi = 0;
  p.rho = rho;
  p.a_out = dunary;
  p.h = dmsg;
  p.edge = edge_weights;
  p.ctx = context;
  p.dedge = dedge_weights;
  p.dctx = dcontext;
  bool first = true;
  for (int it = n_iter - 1; it >= 0; --it) {
    for (int d = s->n_dir - 1; d >= 0; --d) {  // TRWP_backward.cu:337-424
      fill_dirs(s, d, 1, p.dirs, p.block_prefix, &p.n_dirs);
      p.a_in = first ? dcost_final : dunary;  // CostAggregateKernelBack: every g_k starts as dcost
      p.first_touch = (it == n_iter - 1) && (d & 1);
      p.idx_min = msg_min_index + (int64_t)it * s->n_dir * N;
      p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
      launch_bwd<false>(p, st);
      first = false;
    }
  }
  return launch_ok("trwp_backward");
}

int mpl_isgmr_backward(const mpl_shape* s, int enable_sgm, float rho, int n_iter,
                       const float* context, const float* edge_weights, const float* dcost_final,
                       const uint8_t* msg_min_index, const uint8_t* msg_norm_index, float* dunary,
                       float* dcontext, float* dedge_weights, float* dmsg, float* dunary_update,
                       float* dmsg_update, void* stream) {
  (void)dmsg;
  (void)dunary_update;
  int rc = check_shape(s, n_iter);
  if (rc) return rc;
  if (!context || !edge_weights || !dcost_final || !msg_min_index || !msg_norm_index || !dunary ||
      !dcontext || !dedge_weights || !dmsg_update)
    return fail(MPL_EINVAL, "isgmr_backward: null tensor pointer");
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
  p.jacobi = 1;
  p.rho = rho;
  p.du_out = dmsg_update;
  p.edge = edge_weights;
  p.ctx = context;
  p.dedge = dedge_weights;
  p.dctx = dcontext;
  fill_dirs(s, 0, s->n_dir, p.dirs, p.block_prefix, &p.n_dirs);
  for (int it = n_iter - 1; it >= 0; --it) {
    const bool first = (it == n_iter - 1);
    p.gu_in = first ? dcost_final : dmsg_update;  // gu_k = dcost_final for every k at the start
    p.gu_stride = first ? 0 : N;
    p.idx_min = msg_min_index + (int64_t)it * s->n_dir * N;
    p.idx_norm = msg_norm_index + (int64_t)it * s->n_dir * P;
    launch_bwd<true>(p, st);
    isgmr_combine_kernel<<<elementwise_blocks(N), 256, 0, st>>>(
        dmsg_update, s->n_dir, N, rho, dcost_final, factor, first ? 1 : 0, it > 0 ? 1 : 0, dunary);
  }
  return launch_ok("isgmr_backward");
}

}  // extern "C"
