// Scans for small label counts (L <= 32) on gfx950: several chains share one wavefront.
//
// With one chain per wavefront a 21-label problem (the segmentation case) uses a third of the
// lanes.  Here a wavefront walks G = floor(64 / L) chains of one direction at once: lane = g * L + l
// carries label l of the wave's g-th chain, every address is per lane, and the two cross-lane
// patterns of the recurrence work on L-lane segments:
//   * "value of front label fd of my chain" is a ds_bpermute from lane g * L + fd,
//   * min / sum / max over the labels of a chain is a shift-down tree of ds_bpermute steps that
//     ends in the first lane of the segment, followed by one broadcast.
// The step itself is the dense O(L^2) scan of the reference for any context (1-D or 2-D, any sign of
// the edge weights): HorizontalKernel & co., TRWP_forward.cu:82-376, and the reverse scans of
// TRWP_backward.cu:49-275, with the same belief-plane / shared-gradient-plane bookkeeping as the
// one-chain-per-wave kernels (mp_fwd.hip, mp_bwd.hip).
//
// Planes are addressed from their start with 32-bit byte offsets, so a plane (B*H*W*L floats) must
// stay below 2 GiB; larger problems take the one-chain-per-wave kernels.

#include "mp_common.h"

namespace mpl {
namespace {

// Values shared inside a chain's segment of lanes go through LDS: every lane writes its value into
// the slot of its label, and reads the whole segment back with 16-byte loads (all lanes of a segment
// read the same addresses: broadcasts).  One write, one wait and a handful of wide reads replace the
// lane-to-lane exchanges of a reduction tree (six dependent ds_bpermute round trips per reduction at
// 21 labels) or of a loop over the segment's labels (one ds_bpermute per label).  A segment's slots
// start on a 16-byte boundary (Lp = L rounded up to 4 floats); the slots past the last label keep
// the identity of their buffer's operation; lanes without a chain write behind all segments.
typedef int i32x4 __attribute__((ext_vector_type(4)));
constexpr int kRedFloats = 192;  // floats per exchange buffer: G * Lp <= 112, 64 for idle lanes, pad
struct Seg {
  int l;      // label
  int widx;   // where this lane writes
  int rbase;  // first slot of this lane's segment
  int nq;     // 16-byte reads per segment
};

__device__ __forceinline__ Seg make_seg(int lane, int L, int G) {
  Seg s;
  const int g = lane / L;
  const int Lp = (L + 3) & ~3;
  s.l = lane - g * L;
  const bool in = g < G;
  s.widx = in ? g * Lp + s.l : G * Lp + (lane - G * L);
  s.rbase = in ? g * Lp : 0;
  s.nq = Lp / 4;
  return s;
}

// fills the slots past the last label of every segment with the buffer's identity
__device__ __forceinline__ void seg_init(float* buf, float ident, int lane) {
  for (int i = lane; i < kRedFloats; i += kWave) buf[i] = ident;
}

// NQ: compile-time bound of the reads per segment (exactly s.nq when the label count is a
// template constant, 8 otherwise)
template <int NQ, bool EXACT>
__device__ __forceinline__ float seg_min(float* buf, const Seg& s, float x) {
  buf[s.widx] = x;
  const f32x4* q = reinterpret_cast<const f32x4*>(buf + s.rbase);
  float m = INFINITY;
#pragma unroll
  for (int k = 0; k < NQ; ++k) {
    if (!EXACT && k >= s.nq) break;
    const f32x4 v = q[k];
    m = fminf(m, fminf(fminf(v.x, v.y), fminf(v.z, v.w)));
  }
  return m;
}
template <int NQ, bool EXACT>
__device__ __forceinline__ int seg_max(float* buf, const Seg& s, int x) {
  buf[s.widx] = __builtin_bit_cast(float, x);
  const i32x4* q = reinterpret_cast<const i32x4*>(buf + s.rbase);
  int m = -1;
#pragma unroll
  for (int k = 0; k < NQ; ++k) {
    if (!EXACT && k >= s.nq) break;
    const i32x4 v = q[k];
    const int a = v.x > v.y ? v.x : v.y, b = v.z > v.w ? v.z : v.w;
    const int c = a > b ? a : b;
    m = c > m ? c : m;
  }
  return m;
}
template <int NQ, bool EXACT>
__device__ __forceinline__ float seg_sum(float* buf, const Seg& s, float x) {
  buf[s.widx] = x;
  const f32x4* q = reinterpret_cast<const f32x4*>(buf + s.rbase);
  float m = 0.f;
#pragma unroll
  for (int k = 0; k < NQ; ++k) {
    if (!EXACT && k >= s.nq) break;
    const f32x4 v = q[k];
    m += (v.x + v.y) + (v.z + v.w);
  }
  return m;
}
// the values of all labels of the segment: out[c] = value of label c (c < 4 * NQ)
template <int NQ>
__device__ __forceinline__ void seg_all(float* buf, const Seg& s, float x, float (&out)[4 * NQ]) {
  buf[s.widx] = x;
  const f32x4* q = reinterpret_cast<const f32x4*>(buf + s.rbase);
#pragma unroll
  for (int k = 0; k < NQ; ++k) {
    const f32x4 v = q[k];
    out[4 * k] = v.x;
    out[4 * k + 1] = v.y;
    out[4 * k + 2] = v.z;
    out[4 * k + 3] = v.w;
  }
}

// full symmetric context table tab[fd * L + cd] = ctx(cd, fd), TRWP_forward.cu:101-113
__device__ __forceinline__ void fill_table(const float* ctx, int L, int ctx2d, int lane, float* tab) {
  for (int i = lane; i < L * L; i += kWave) {
    const int fd = i / L, cd = i - fd * L;
    const int lo = cd < fd ? cd : fd, hi = cd < fd ? fd : cd;
    tab[i] = ctx[ctx2d ? lo * L + hi : hi - lo];
  }
}

// The chains of this wavefront: direction, and per lane the first pixel (index over the whole
// batch), the number of pixels (0 for idle lanes) and the pixel stride.
struct PackedChains {
  int dir, pstep, n, pix0, n_max;
  bool on;
};

template <typename Params>
__device__ __forceinline__ PackedChains locate_packed(const Params& p, int lane, int L, int G) {
  int di = 0;
  while (di + 1 < p.n_dirs && (int)blockIdx.x >= p.block_prefix[di + 1]) ++di;
  PackedChains c;
  c.dir = p.dirs[di];
  const int wave = (int)blockIdx.x - p.block_prefix[di];
  const DirGeom geo = make_dir(c.dir, p.H, p.W);
  const int g = lane / L;
  const int64_t total = (int64_t)p.B * geo.n_chains;
  const int64_t idx = (int64_t)wave * G + g;
  c.on = (g < G) && (idx < total);
  c.n = 0;
  c.pix0 = 0;
  if (c.on) {
    const int bv = (int)(idx / geo.n_chains);
    const int ch = (int)(idx - (int64_t)bv * geo.n_chains);
    int h0, w0;
    chain_start(geo, p.H, p.W, ch, &h0, &w0, &c.n);
    c.pix0 = bv * p.H * p.W + h0 * p.W + w0;
  }
  c.pstep = geo.hs * p.W + geo.ws;
  c.n_max = (int)(-wave_min(-(float)c.n));
  return c;
}

__device__ __forceinline__ float ldf(rsrc_t r, unsigned off) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, MPL_LD_AUX));
}
__device__ __forceinline__ void stf(rsrc_t r, unsigned off, float v) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, (int)off, 0, MPL_ST_AUX);
}

struct PixPF {
  float s, md, mi, w;
};

// LT > 0: label count known at compile time (21): front-label loop unrolled, context column in
// registers.
template <bool TRAIN, bool JACOBI, int LT>
__global__ void __launch_bounds__(kWave) packed_fwd_kernel(const SweepParams p) {
  extern __shared__ float smem[];
  float* xa = smem;                  // exchange buffers (see Seg): beliefs a,
  float* xm = xa + kRedFloats;       // normalisation minimum,
  float* xi = xm + kRedFloats;       // its label
  float* tab = xi + kRedFloats;      // L * L
  const int L = LT > 0 ? LT : p.L;
  const int G = p.pack;
  const int lane = threadIdx.x;
  const PackedChains ch0 = locate_packed(p, lane, L, G);
  const Seg sg = make_seg(lane, L, G);
  constexpr int NQ = LT > 0 ? (LT + 3) / 4 : 8;
  constexpr bool EXACT = LT > 0;
  seg_init(xa, 0.f, lane);
  seg_init(xm, INFINITY, lane);
  seg_init(xi, __builtin_bit_cast(float, -1), lane);
  fill_table(p.ctx, L, p.ctx2d, lane, tab);
  __syncthreads();
  if (!JACOBI && !p.pair_q && ch0.n_max < 2) return;

  const int64_t P = (int64_t)p.B * p.H * p.W;
  const int64_t N = P * L;
  // Gauss-Seidel, at most one wavefront per SIMD (p.fused_pair): after the sweep of dirs[0] the
  // wavefront sweeps the opposite direction over the same pixels in reverse (see mp_fwd.hip)
  const int halves = (!JACOBI && p.fused_pair) ? 2 : 1;
#pragma clang loop unroll(disable)
  for (int half = 0; half < halves; ++half) {
  PackedChains ch = ch0;
  bool skip_s_store = p.skip_s_store != 0;
  if (half) {
    ch.dir = ch0.dir ^ 1;
    ch.pix0 = ch0.pix0 + (ch0.n - 1) * ch0.pstep;
    ch.pstep = -ch0.pstep;
    skip_s_store = p.skip_s_store2 != 0;
    wait_vmem<0>();
    __syncthreads();
  }
  const int dir = ch.dir;
  const int plane_bytes = (int)(N * 4);
  const bool md_zero = !JACOBI && p.first_iter && p.desc != nullptr && p.desc->msg_nonzero == 0;
  const bool mi_zero = md_zero && (dir & 1) == 0;
  const bool pair_first = !JACOBI && p.pair_q && (dir & 1) == 0;   // see mp_fwd.hip
  const bool pair_second = !JACOBI && p.pair_q && (dir & 1) == 1;
  const int udir = p.u_pair_share ? (dir & ~1) : dir;
  const rsrc_t dS = make_rsrc(JACOBI ? p.msg_in + (int64_t)udir * p.u_stride : p.belief, plane_bytes);
  const rsrc_t dMd = make_rsrc(p.msg_in + (int64_t)dir * N, (JACOBI || md_zero) ? 0 : plane_bytes);
  const rsrc_t dMdRing = make_rsrc(p.msg_in + (int64_t)dir * N,
                                   (JACOBI || md_zero || pair_second) ? 0 : plane_bytes);
  const rsrc_t dMi = make_rsrc(p.msg_in + (int64_t)(dir ^ 1) * N, (JACOBI || mi_zero) ? 0 : plane_bytes);
  const rsrc_t dMo = make_rsrc(p.msg_out + (int64_t)dir * N, plane_bytes);
  const rsrc_t dSo = make_rsrc(JACOBI ? nullptr : p.belief_out, (JACOBI || skip_s_store) ? 0 : plane_bytes);
  const rsrc_t dW = make_rsrc(p.edge + (int64_t)dir * P, (int)(P * 4));
  const rsrc_t dImin = make_rsrc(TRAIN ? p.idx_min + (int64_t)dir * N : nullptr, TRAIN ? (int)N : 0);
  const rsrc_t dInorm = make_rsrc(TRAIN ? p.idx_norm + (int64_t)dir * P : nullptr, TRAIN ? (int)P : 0);
  const float rho = p.rho;
  const float inf = INFINITY;
  const int l = sg.l;
  const bool on = ch.on;
  const int n = ch.n;

  float tcol[LT > 0 ? LT : 1];
  if (LT > 0) {
#pragma unroll
    for (int fd = 0; fd < LT; ++fd) tcol[fd] = tab[fd * LT + l];
  }

  int ld_pix = ch.pix0, ld_t = 0;
  auto load_next = [&]() {
    PixPF r;
    const bool act = on && ld_t < n;
    const unsigned eo = act ? (unsigned)(ld_pix * L + l) * 4u : (unsigned)kDeadOffset;
    r.s = ldf(dS, eo);
    if (!JACOBI) {
      r.md = ldf(ld_t == 0 ? dMd : dMdRing, eo);
      r.mi = ldf(dMi, eo);
    } else {
      r.md = r.mi = 0.f;
    }
    r.w = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                        dW, act ? ld_pix * 4 : kDeadOffset, 0, 0));
    ld_pix += ch.pstep;
    ld_t += 1;
    return r;
  };

  float prev = 0.f, uf;
  {
    const PixPF p0 = load_next();
    MPL_ORDER_LOADS();  // (the chain start's loads stay ahead of the ring's)
    const float t0 = pair_second ? p0.s + p0.mi : p0.s - p0.md;
    const float un = JACOBI ? p0.s : fmaf(t0, rho, -p0.mi);
    uf = on ? un : inf;
    if (!JACOBI && p.pair_q)  // convert the belief plane at the chain start as well
      stf(dSo, (on && n >= 1) ? (unsigned)(ch.pix0 * L + l) * 4u : (unsigned)kDeadOffset,
          pair_second ? t0 + p0.md : t0 - p0.mi);
    if (JACOBI || p.zero_start)  // the chain start is written with the zeros it keeps
      stf(dMo, (on && n >= 1) ? (unsigned)(ch.pix0 * L + l) * 4u : (unsigned)kDeadOffset, 0.f);
  }

  constexpr int kOps = (JACOBI ? 1 : 3) + 1 + (JACOBI ? 1 : 2) + (TRAIN ? 2 : 0);
  constexpr int D = ring_depth(kOps);
  // Gauss-Seidel launches have few wavefronts per SIMD (one direction each): two banks of
  // prefetched pixels, filled and used in turn, so that no register is moved and no wait drains
  // the queue.  Jacobi launches (all directions at once) have many, which hide such waits, and
  // gain more from the registers a single bank saves (measured at 8256 chains: 0.60 against 0.66 ms).
  constexpr bool kTwoBanks = !JACOBI;
  PixPF ring[D], ring2[kTwoBanks ? D : 1];
#pragma unroll
  for (int u = 0; u < D; ++u) {
    ring[u] = load_next();
    // keeps the pixels' loads in this order: the compiler's own waits in the loop are sized for
    // the order it sees here, and a later pixel's loads placed first would make them drain the queue
    MPL_ORDER_LOADS();
  }

  int st_pix = ch.pix0 + ch.pstep;
  auto step = [&](const PixPF& px, const int t) __attribute__((always_inline)) {
      const bool live = on && t < n;
      const float tt = pair_second ? px.s + px.mi : px.s - px.md;
      const float x = JACOBI ? px.s : fmaf(tt, rho, -px.mi);  // UpdateUnaryKernel, :70-78
      const float un = on ? x : inf;
      const float w = px.w;
      const float a = fmaf(rho, prev, uf);
      // v[cd] = min_fd a[fd] + w * ctx(cd, fd), largest fd on ties (TRWP_forward.cu:127-153)
      float best = inf;
      int arg = L - 1;
      if constexpr (LT > 0) {
        float av[4 * NQ];  // a of every label of this lane's chain
        seg_all<NQ>(xa, sg, a, av);
#pragma unroll
        for (int fd = LT - 1; fd >= 0; --fd) {
          const float val = fmaf(w, tcol[fd], av[fd]);
          if (TRAIN) {
            const bool take = (fd == LT - 1) || (val < best);
            best = take ? val : best;
            arg = take ? fd : arg;
          } else {
            best = fminf(best, val);
          }
        }
      } else {
        xa[sg.widx] = a;
#pragma unroll 4
        for (int fd = L - 1; fd >= 0; --fd) {
          const float val = fmaf(w, tab[fd * L + l], xa[sg.rbase + fd]);
          if (TRAIN) {
            const bool take = (fd == L - 1) || (val < best);
            best = take ? val : best;
            arg = take ? fd : arg;
          } else {
            best = fminf(best, val);
          }
        }
      }
      const float nmin = seg_min<NQ, EXACT>(xm, sg, on ? best : inf);  // MsgNormNaive, commonCUDA.cuh:92-129
      const float m = best - nmin;
      prev = on ? m : 0.f;
      uf = un;
      const unsigned eo = live ? (unsigned)(st_pix * L + l) * 4u : (unsigned)kDeadOffset;
      stf(dMo, eo, m);
      if (!JACOBI) stf(dSo, eo, pair_first ? tt - px.mi : tt + m);
      if (TRAIN) {
        __builtin_amdgcn_raw_buffer_store_b8((unsigned char)arg, dImin,
                                             live ? st_pix * L + l : kDeadOffset, 0, MPL_ST_AUX);
        const int nidx = seg_max<NQ, EXACT>(xi, sg, (on && best == nmin) ? l : -1);  // largest label on ties
        __builtin_amdgcn_raw_buffer_store_b8((unsigned char)nidx, dInorm,
                                             (live && l == 0) ? st_pix : kDeadOffset, 0, 0);
      }
      st_pix += ch.pstep;
  };
  if constexpr (kTwoBanks) {
    for (int t0 = 1; t0 < ch.n_max; t0 += 2 * D) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        // the loads of this ring slot were followed by at most D-1 steps' worth of memory operations
        wait_vmem<(D - 1) * kOps>();
        const PixPF px = ring[u];
        ring2[u] = load_next();
        MPL_ORDER_LOADS();  // the next pixel's loads go out before this step's work
        step(px, t0 + u);
      }
      if (t0 + D >= ch.n_max) break;  // wave-uniform
#pragma unroll
      for (int u = 0; u < D; ++u) {
        wait_vmem<(D - 1) * kOps>();
        const PixPF px = ring2[u];
        ring[u] = load_next();
        MPL_ORDER_LOADS();
        step(px, t0 + D + u);
      }
    }
  } else {
    for (int t0 = 1; t0 < ch.n_max; t0 += D) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        wait_vmem<(D - 1) * kOps>();
        const PixPF px = ring[u];
        ring[u] = load_next();
        step(px, t0 + u);
      }
    }
  }
  }  // both sweeps of a fused pair
}

struct PixPB {
  float a, hd, hi;
  int fd, nidx;
  float w, de;
};

// GRAD: bit 0 = dedge_weights is wanted, bit 1 = dcontext is wanted
template <bool JACOBI, int LT, int GRAD>
__global__ void __launch_bounds__(kWave) packed_bwd_kernel(const BackParams p) {
  constexpr bool DE = (GRAD & 1) != 0, DC = (GRAD & 2) != 0;
  extern __shared__ float smem[];
  const int L = LT > 0 ? LT : p.L;
  const int G = p.pack;
  float* xg = smem;                  // exchange buffers (see Seg): gradients g,
  float* xf = xg + kRedFloats;       // argmin labels,
  float* xs = xf + kRedFloats;       // the two sums
  float* xd = xs + kRedFloats;
  float* tab = xd + kRedFloats;      // L * L
  float* pairs = tab + L * L;        // G tables of L * L: dcontext per (cd, fd) pair and chain slot
  const int lane = threadIdx.x;
  const PackedChains ch0 = locate_packed(p, lane, L, G);
  const Seg sg = make_seg(lane, L, G);
  constexpr int NQ = LT > 0 ? (LT + 3) / 4 : 8;
  constexpr bool EXACT = LT > 0;
  seg_init(xg, 0.f, lane);
  seg_init(xf, __builtin_bit_cast(float, -1), lane);
  seg_init(xs, 0.f, lane);
  seg_init(xd, 0.f, lane);
  if (DE) fill_table(p.ctx, L, p.ctx2d, lane, tab);
  if (DC)
    for (int i = lane; i < G * L * L; i += kWave) pairs[i] = 0.f;
  __syncthreads();

  const int64_t P = (int64_t)p.B * p.H * p.W;
  const int64_t N = P * L;
  const int plane_bytes = (int)(N * 4);
  const bool same = p.same_label != 0;
  // Gauss-Seidel, at most one wavefront per SIMD (p.fused_pair): the walk for the odd direction,
  // then the one for the even direction over the same pixels in reverse (see mp_bwd.hip)
  const int halves = (!JACOBI && p.fused_pair) ? 2 : 1;
#pragma clang loop unroll(disable)
  for (int half = 0; half < halves; ++half) {
  PackedChains ch = ch0;
  bool first_touch = p.first_touch != 0, inv_a = p.inv_from_a != 0;
  bool skip_hd_store = p.skip_hd_store != 0, skip_hi_store = p.skip_hi_store != 0;
  const float* a_in = p.a_in;
  if (half) {
    ch.dir = ch0.dir ^ 1;
    ch.pix0 = ch0.pix0 + (ch0.n - 1) * ch0.pstep;
    ch.pstep = -ch0.pstep;
    first_touch = false;
    inv_a = true;
    skip_hd_store = skip_hi_store = p.skip_h2 != 0;
    a_in = p.a_out;
    wait_vmem<0>();
    __syncthreads();
  }
  const int dir = ch.dir;
  const bool read_h = !JACOBI && !first_touch;
  const bool inv_from_a = !JACOBI && inv_a;
  const int gdir = p.gu_pair_share ? (dir & ~1) : dir;
  const rsrc_t dA = make_rsrc(JACOBI ? p.gu_in + (int64_t)gdir * p.gu_stride : a_in, plane_bytes);
  const rsrc_t dAo = make_rsrc(JACOBI ? p.du_out + (int64_t)dir * N : p.a_out, plane_bytes);
  float* hbase = JACOBI ? p.du_out : p.h;
  const rsrc_t dHdIn = make_rsrc(hbase + (int64_t)dir * N, read_h ? plane_bytes : 0);
  const rsrc_t dHiIn = make_rsrc(hbase + (int64_t)(dir ^ 1) * N, (read_h && !inv_from_a) ? plane_bytes : 0);
  const rsrc_t dHdOut = make_rsrc(hbase + (int64_t)dir * N, (JACOBI || skip_hd_store) ? 0 : plane_bytes);
  const rsrc_t dHiOut = make_rsrc(hbase + (int64_t)(dir ^ 1) * N, (JACOBI || skip_hi_store) ? 0 : plane_bytes);
  const rsrc_t dImin = make_rsrc(p.idx_min + (int64_t)dir * N, (int)N);
  const rsrc_t dInorm = make_rsrc(p.idx_norm + (int64_t)dir * P, (int)P);
  const rsrc_t dW = make_rsrc(p.edge + (int64_t)dir * P, (int)(P * 4));
  const rsrc_t dDe = make_rsrc(DE ? p.dedge + (int64_t)dir * P : nullptr, DE ? (int)(P * 4) : 0);
  const float rho = p.rho;
  const int l = sg.l;
  const bool on = ch.on;
  const int n = ch.n;
  float* my_pairs = pairs + (lane / L < G ? lane / L : 0) * L * L + l * L;  // row of this label

  // every chain is walked from its own last pixel: step s visits t = n - 1 - s
  int ld_pix = ch.pix0 + (n - 1) * ch.pstep, ld_t = n - 1;
  auto load_next = [&]() {
    PixPB r;
    const bool act = on && ld_t >= 0;
    const unsigned eo = act ? (unsigned)(ld_pix * L + l) * 4u : (unsigned)kDeadOffset;
    r.a = ldf(dA, eo);
    if (!JACOBI) {
      r.hd = ldf(dHdIn, eo);
      r.hi = ldf(dHiIn, eo);
      if (inv_from_a) r.hi = -r.a;
    } else {
      r.hd = r.hi = 0.f;
    }
    r.fd = __builtin_amdgcn_raw_buffer_load_b8(dImin, act ? ld_pix * L + l : kDeadOffset, 0, MPL_LD_AUX);
    r.nidx = __builtin_amdgcn_raw_buffer_load_b8(dInorm, act ? ld_pix : kDeadOffset, 0, 0);
    r.w = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                        dW, act ? ld_pix * 4 : kDeadOffset, 0, 0));
    r.de = 0.f;
    if (DE)
      r.de = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                           dDe, (act && l == 0) ? ld_pix * 4 : kDeadOffset, 0, 0));
    ld_pix -= ch.pstep;
    ld_t -= 1;
    return r;
  };

  constexpr int kOps = (JACOBI ? 1 : 3) + 3 + (DE ? 1 : 0) + (JACOBI ? 1 : 3) + (DE ? 1 : 0);
  constexpr int D = ring_depth(kOps);
  PixPB ring[D];
#pragma unroll
  for (int u = 0; u < D; ++u) {
    ring[u] = load_next();
    // keeps the pixels' loads in this order: the compiler's own waits in the loop are sized for
    // the order it sees here, and a later pixel's loads placed first would make them drain the queue
    MPL_ORDER_LOADS();
  }

  float sc = 0.f;  // dU of the current pixel: what the previous step scattered into it
  int st_pix = ch.pix0 + (n - 1) * ch.pstep;
  for (int s0 = 0; s0 < ch.n_max; s0 += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int t = n - 1 - (s0 + u);  // per lane
      const bool here = on && t >= 0;  // this lane's chain has a pixel at this step
      wait_vmem<(D - 1) * kOps>();
      const PixPB px = ring[u];
      ring[u] = load_next();
      // gradient w.r.t. the normalised message of this pixel (none at the chain start, t == 0)
      const bool edge = on && t >= 1;
      float g = edge ? fmaf(rho, sc, JACOBI ? px.a : px.a + px.hd) : 0.f;
      const float tot = seg_sum<NQ, EXACT>(xs, sg, g);  // MsgNormNaiveBack, commonCUDA.cuh:131-145
      if (edge && l == px.nidx) g -= tot;
      const int fd = px.fd;
      // dU[q, f] = sum of g[c] over the labels c of this chain whose argmin is f
      float scn = 0.f;
      if constexpr (LT > 0) {
        float gv[4 * NQ], fv[4 * NQ];  // gradient and argmin label of every label of the chain
        seg_all<NQ>(xg, sg, g, gv);
        seg_all<NQ>(xf, sg, __builtin_bit_cast(float, fd), fv);
#pragma unroll
        for (int c = 0; c < LT; ++c) scn += (__builtin_bit_cast(int, fv[c]) == l) ? gv[c] : 0.f;
      } else {
        xg[sg.widx] = g;
        xf[sg.widx] = __builtin_bit_cast(float, fd);
#pragma unroll 4
        for (int c = 0; c < L; ++c) {
          const float gc = xg[sg.rbase + c];
          const int fc = __builtin_bit_cast(int, xf[sg.rbase + c]);
          scn += (fc == l) ? gc : 0.f;
        }
      }
      // dedge_weights[p] += ctx(cd, fd) * g;  dcontext[(cd, fd)] += w * g for cd != fd
      // (TRWP_backward.cu:109-112)
      const int fdc = edge ? fd : 0;
      float det = 0.f;
      if (DE) det = seg_sum<NQ, EXACT>(xd, sg, tab[fdc * L + l] * g);
      if (DC && edge && (same || fdc != l)) my_pairs[fdc] = fmaf(px.w, g, my_pairs[fdc]);
      const unsigned eo = here ? (unsigned)(st_pix * L + l) * 4u : (unsigned)kDeadOffset;
      if (JACOBI) {
        stf(dAo, eo, sc);
      } else {
        const float an = fmaf(rho, sc, px.a);  // g_k += rho * dU for every k, dunary too
        stf(dAo, eo, an);
        stf(dHdOut, eo, -an);          // g_dir = 0 after its sweep
        stf(dHiOut, eo, px.hi - sc);   // g_inv -= dU
      }
      if (DE)
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, px.de + det), dDe,
                                              (edge && l == 0) ? st_pix * 4 : kDeadOffset, 0, 0);
      sc = here ? scn : 0.f;
      st_pix -= ch.pstep;
    }
  }
  }  // both walks of a fused pair
  if (!DC) return;
  __syncthreads();
  // fold the pair tables of all chain slots into dcontext's bins (the pairs with cd == fd were
  // only collected when the caller asked for them)
  if (!p.ctx2d) {
    if (lane < L) {
      float acc = 0.f;
      for (int g2 = 0; g2 < G; ++g2)
        for (int c = 0; c < L; ++c) {
          if (c + lane < L) acc += pairs[g2 * L * L + c * L + c + lane];
          if (lane >= 1 && c - lane >= 0) acc += pairs[g2 * L * L + c * L + c - lane];
        }
      if (acc != 0.f) atomicAdd(&p.dctx[lane], acc);
    }
  } else {
    for (int i = lane; i < L * L; i += kWave) {
      const int c = i / L, f = i - c * L;
      if (c > f) continue;
      float v = 0.f;
      for (int g2 = 0; g2 < G; ++g2)
        v += pairs[g2 * L * L + i] + (c < f ? pairs[g2 * L * L + f * L + c] : 0.f);
      if (v != 0.f) atomicAdd(&p.dctx[i], v);
    }
  }
}

// prefix sums of wavefronts per direction for G chains per wavefront
template <typename Params>
Params with_wave_prefix(const Params& p, int G) {
  Params q = p;
  q.pack = G;
  q.block_prefix[0] = 0;
  for (int i = 0; i < p.n_dirs; ++i) {
    const int64_t chains = (int64_t)p.B * make_dir(p.dirs[i], p.H, p.W).n_chains;
    q.block_prefix[i + 1] = q.block_prefix[i] + (int)((chains + G - 1) / G);
  }
  return q;
}

}  // namespace

int packed_chains_per_wave(int B, int H, int W, int L, bool ctx2d, int64_t chains, bool always) {
  if (L > kPackedMaxL) return 0;
  if ((int64_t)B * H * W * L * 4 >= (int64_t)kDeadOffset) return 0;  // 32-bit plane offsets
  // A packed step serves up to 64 / L chains but is longer than the step of a wavefront with one
  // chain (every value shared inside a chain crosses LDS, and it scans all L front labels per
  // label whatever the table), so it pays once the launch has more chains than the chip has SIMDs,
  // for a dense table.  Measured, fwd+bwd, packed against one chain per wavefront:
  //  * 21 labels, 2-D table, 4 x H x H: TRWP with 1032 chains per launch 6.2 against 5.4 ms, 1548
  //    chains 9.3 against 8.5, 1804 chains 10.8 against 10.2, but 2064 chains (a third wavefront on
  //    some SIMDs) 12.6 against 15.0; ISGMR with 1536 chains 0.88 against 0.85, 2064 chains 1.12
  //    against 1.28, 8256 chains 6.9 against 11.4;
  //  * 1-D tables, ISGMR, 3 iterations: min(k, 3) with 16 / 32 labels and 1280 chains 2.0 / 3.7
  //    against 0.73 / 0.88 ms; dense with 16 / 32 labels, 1280 chains 2.0 / 3.7 against 1.3 / 2.3
  //    and 10240 chains 5.2 / 15.0 against 9.7 / 18.2; 8 labels, 5120 chains, dense 1.42 against
  //    1.62 and min(k, 3) 1.42 against 1.36; 4 labels, 5120 chains, dense 0.98 against 1.34;
  //    min(k, 3) with 16 labels: 5120 chains 4.6 against 3.3, 10240 chains 5.2 against 6.4, 40960
  //    chains 17.0 against 25.3 (TRWP, 10240 chains per launch: 21.1 against 25.2); with 12 labels
  //    and 10240 chains 4.3 against 6.4; with 32 labels and 10240 chains 15.1 against 10.4.  With
  //    8 directions, whose diagonal chains are short, on 300 x 400: 8 labels, batch 1 (4196 chains)
  //    1.05 against 0.61, batch 2 with 5 labels (8392 chains) 0.99 against 1.22, batch 4 (16784
  //    chains) 1.40 against 2.02; 16 labels, batch 2 (8392 chains) 1.81 against 1.42, batch 4 2.11
  //    against 2.56.
  if (!always) {
    const LaunchPolicy& pol = launch_policy();
    if (ctx2d) {
      if (chains < (L == 21 ? pol.packed_min_chains21 : pol.packed_min_chains)) return 0;
    } else {
      if (L > 16 || chains < (L <= 8 ? pol.packed_min_chains_1d8 : pol.packed_min_chains_1d16)) return 0;
    }
  }
  int G = kWave / L;
  return G > 16 ? 16 : G;
}

void launch_packed_fwd(const SweepParams& p0, bool train, bool jacobi, int G, hipStream_t st) {
  const SweepParams p = with_wave_prefix(p0, G);
  const int blocks = p.block_prefix[p.n_dirs];
  const size_t lds = sizeof(float) * (3 * kRedFloats + p.L * p.L);
#define MPL_PACKED_FWD(LT)                                                                 \
  do {                                                                                     \
    if (train) {                                                                           \
      if (jacobi)                                                                          \
        packed_fwd_kernel<true, true, LT><<<blocks, kWave, lds, st>>>(p);                  \
      else                                                                                 \
        packed_fwd_kernel<true, false, LT><<<blocks, kWave, lds, st>>>(p);                 \
    } else {                                                                               \
      if (jacobi)                                                                          \
        packed_fwd_kernel<false, true, LT><<<blocks, kWave, lds, st>>>(p);                 \
      else                                                                                 \
        packed_fwd_kernel<false, false, LT><<<blocks, kWave, lds, st>>>(p);                \
    }                                                                                      \
  } while (0)
  if (p.L == 21)
    MPL_PACKED_FWD(21);
  else
    MPL_PACKED_FWD(0);
#undef MPL_PACKED_FWD
}

void launch_packed_bwd(const BackParams& p0, bool jacobi, int G, hipStream_t st) {
  const BackParams p = with_wave_prefix(p0, G);
  const int blocks = p.block_prefix[p.n_dirs];
  const size_t lds = sizeof(float) * (4 * kRedFloats + p.L * p.L * (1 + G));
#define MPL_PACKED_BWD(GRAD)                                                  \
  do {                                                                        \
    if (p.L == 21) {                                                          \
      if (jacobi)                                                             \
        packed_bwd_kernel<true, 21, GRAD><<<blocks, kWave, lds, st>>>(p);     \
      else                                                                    \
        packed_bwd_kernel<false, 21, GRAD><<<blocks, kWave, lds, st>>>(p);    \
    } else {                                                                  \
      if (jacobi)                                                             \
        packed_bwd_kernel<true, 0, GRAD><<<blocks, kWave, lds, st>>>(p);      \
      else                                                                    \
        packed_bwd_kernel<false, 0, GRAD><<<blocks, kWave, lds, st>>>(p);     \
    }                                                                         \
  } while (0)
  switch ((p.dedge != nullptr ? 1 : 0) | (p.dctx != nullptr ? 2 : 0)) {
    case 0: MPL_PACKED_BWD(0); break;
    case 1: MPL_PACKED_BWD(1); break;
    case 2: MPL_PACKED_BWD(2); break;
    default: MPL_PACKED_BWD(3); break;
  }
#undef MPL_PACKED_BWD
}

}  // namespace mpl
