// Soft-weighted TRWP for gfx950 (forward and reverse scans): the min over front labels of the hard
// layer is replaced by the expectation of the dual under softmin weights.  Follows
// DynamicProgramming / DynamicProgrammingBack of the reference
// (MPLayers/TRWP_hard_soft/TRWP_forward_soft.cu:9-117, TRWP_backward_soft.cu:9-129):
//     dual[cd, fd] = U[q, fd] + rho * m[q, fd] + w[p] * ctx(cd, fd)
//     prob[cd, fd] = softmax_fd(-dual[cd, :]),   soft[cd] = sum_fd prob * dual
//     m[p, :]      = soft - min_cd soft                       (largest cd on ties)
// Training keeps the whole (L, L) block of duals per pixel, direction and iteration
// (msg_edge_label; even directions store [fd][cd], odd ones [cd][fd]); the reverse scan rebuilds
// prob from it:
//     ddual[cd, fd] = g[cd] * prob * (1 - dual + soft[cd])
//     dU[q, fd] += sum_cd ddual;  dedge[p] += sum ctx * ddual;  dcontext[ctx index] += w[p] * ddual
//
// Mapping: one wavefront per chain, one label per lane (L <= 64), pixel planes prefetched through a
// register ring as in the hard kernels.  The (L, L) block goes through LDS so that global memory
// sees it as T = ceil(L*L/64) coalesced dword accesses per lane; T is a template bucket so that the
// number of memory instructions per step is a compile-time constant.

#include "mp_common.h"

namespace mpl {
namespace {

__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }

struct PixSF {
  float s, md, mi, w;
};

// full symmetric context table tab[fd * L + cd] = ctx(cd, fd): TRWP_forward_soft.cu:55-59
__device__ __forceinline__ void fill_table(const float* ctx, int L, int ctx2d, int lane, float* tab) {
  for (int i = lane; i < L * L; i += kWave) {
    const int fd = i / L, cd = i - fd * L;
    const int lo = cd < fd ? cd : fd, hi = cd < fd ? fd : cd;
    tab[i] = ctx[ctx2d ? lo * L + hi : hi - lo];
  }
}

// LT > 0: the label count is known at compile time (the segmentation case, 21 labels): the loops
// over front labels are unrolled and the lane's column of the context table lives in registers.
template <bool TRAIN, int T, int LT>
__global__ void __launch_bounds__(kWave) soft_fwd_kernel(const SweepParams p) {
  extern __shared__ float smem[];
  const int L = LT > 0 ? LT : p.L, LL = L * L;
  float* tab = smem;        // LL floats
  float* tile = smem + LL;  // max(LL, 64 * T) floats: the pixel's block of duals
  const int lane = threadIdx.x;
  const ChainCtx ch = locate_chain(p);
  if (ch.n < 2) return;  // nothing to write
  fill_table(p.ctx, L, p.ctx2d, lane, tab);
  __syncthreads();

  const int64_t HW = (int64_t)p.H * p.W;
  const int64_t P = (int64_t)p.B * HW;
  const int64_t N = P * L;
  const int dir = ch.dir;
  const int64_t img_p = (int64_t)ch.bv * HW;
  const int64_t img_e = img_p * L;
  const int vbytes = L * 4;
  const float* __restrict__ bS = p.belief + img_e;
  const float* __restrict__ bMd = p.msg_in + (int64_t)dir * N + img_e;
  const float* __restrict__ bMi = p.msg_in + (int64_t)(dir ^ 1) * N + img_e;
  float* __restrict__ bMo = p.msg_out + (int64_t)dir * N + img_e;
  float* __restrict__ bSo = p.belief_out + img_e;
  float* __restrict__ bBlk = TRAIN ? p.edge_label + ((int64_t)dir * P + img_p) * LL : nullptr;
  const int img_bytes_p = (int)(HW * 4 > 0x7fffffff ? 0x7fffffff : HW * 4);
  const rsrc_t dW = make_rsrc(p.edge + (int64_t)dir * P + img_p, img_bytes_p);
  const rsrc_t dInorm = make_rsrc(TRAIN ? p.idx_norm + (int64_t)dir * P + img_p : nullptr,
                                  TRAIN ? (int)HW : 0);
  const float rho = p.rho;
  const float inf = INFINITY;
  const int foff = lane * 4;
  const int n = ch.n;
  const bool valid = lane < L;
  const int col = valid ? lane : L - 1;  // keeps the table reads of idle lanes in range
  const bool even = (dir & 1) == 0;
  float tcol[LT > 0 ? LT : 1];  // ctx(cd = lane, fd)
  if (LT > 0) {
#pragma unroll
    for (int fd = 0; fd < LT; ++fd) tcol[fd] = tab[fd * L + col];
  }
  const int wstep = even ? L : 1;             // address step of the front label inside the block
  const int wbase = even ? lane : lane * L;   // address of (cd = lane, fd = 0)

  const int last_p = ch.pix0 + (n - 1) * ch.pstep;
  int ld_p = ch.pix0;
  int ld_t = 0;
  auto load_next = [&]() {
    PixSF r;
    const unsigned pp = (unsigned)uniform_i(ld_t < n ? ld_p : last_p);
    const unsigned so = pp * (unsigned)vbytes;
    const int nrec = (int)(so + (unsigned)vbytes);
    float t1[1];
    buf_load<1, true>(make_rsrc(bS, nrec), foff, so, t1);
    r.s = t1[0];
    buf_load<1, true>(make_rsrc(bMd, nrec), foff, so, t1);
    r.md = t1[0];
    buf_load<1, true>(make_rsrc(bMi, nrec), foff, so, t1);
    r.mi = t1[0];
    r.w = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dW, (int)(pp * 4u), 0, 0));
    ld_p += ch.pstep;
    ld_t += 1;
    return r;
  };

  float prev = 0.f, uf;
  {
    const PixSF p0 = load_next();
    const float un = fmaf(p0.s - p0.md, rho, -p0.mi);
    uf = valid ? un : inf;
  }

  constexpr int kOps = 4 + 2 + (TRAIN ? 1 + T : 0);
  constexpr int D = ring_depth(kOps);
  PixSF ring[D];
#pragma unroll
  for (int u = 0; u < D; ++u) ring[u] = load_next();

  int st_p = ch.pix0 + ch.pstep;
  for (int t0 = 1; t0 < n; t0 += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int t = t0 + u;
      const bool live = t < n;
      wait_vmem<(D - 1) * kOps>();
      const PixSF px = ring[u];
      ring[u] = load_next();
      const float tt = px.s - px.md;
      const float un = valid ? fmaf(tt, rho, -px.mi) : inf;  // UpdateUnaryKernelSoft, :161-181
      const float w = uniform_f(px.w);
      const float a = fmaf(rho, prev, uf);  // lane = front label
      // pass 1: minimum of the duals of this lane's label; the block goes to LDS
      float mn = inf;
      float se = 0.f, sd = 0.f;
      if constexpr (LT > 0) {
        float dual[LT];
#pragma unroll
        for (int fd = 0; fd < LT; ++fd) {
          dual[fd] = fmaf(w, tcol[fd], readlane_f(a, fd));
          mn = fminf(mn, dual[fd]);
        }
        if (TRAIN && valid) {  // one predicated region for the whole column, not one per store
#pragma unroll
          for (int fd = 0; fd < LT; ++fd) tile[wbase + fd * wstep] = dual[fd];
        }
        // pass 2: softmin weights and the expected dual
#pragma unroll
        for (int fd = 0; fd < LT; ++fd) {
          const float e = fast_exp(mn - dual[fd]);
          se += e;
          sd = fmaf(e, dual[fd], sd);
        }
      } else {
#pragma unroll 4
        for (int fd = 0; fd < L; ++fd) {
          const float dual = fmaf(w, tab[fd * L + col], readlane_f(a, fd));
          mn = fminf(mn, dual);
          if (TRAIN && valid) tile[wbase + fd * wstep] = dual;
        }
#pragma unroll 4
        for (int fd = 0; fd < L; ++fd) {
          const float dual = fmaf(w, tab[fd * L + col], readlane_f(a, fd));
          const float e = fast_exp(mn - dual);
          se += e;
          sd = fmaf(e, dual, sd);
        }
      }
      const float soft = sd / se;
      const float nmin = wave_min(valid ? soft : inf);
      const float m = soft - nmin;
      const float sn = tt + m;
      prev = valid ? m : 0.f;
      uf = un;
      const unsigned sp = (unsigned)uniform_i(st_p);
      const unsigned so = sp * (unsigned)vbytes;
      const int nrec = live ? (int)(so + (unsigned)vbytes) : 0;
      const float m1[1] = {m}, s1[1] = {sn};
      buf_store<1, true>(make_rsrc(bMo, nrec), foff, so, m1);
      buf_store<1, true>(make_rsrc(bSo, nrec), foff, so, s1);
      if (TRAIN) {
        const bool pr[1] = {valid && (soft == nmin)};
        const int nidx = last_label<1>(pr, L - 1);
        __builtin_amdgcn_raw_buffer_store_b8((unsigned char)nidx, dInorm,
                                             live ? (int)sp : kDeadOffset, 0, 0);
        // the block as T coalesced dwords per lane; elements past L*L fall outside the descriptor
        const rsrc_t dBlk = make_rsrc(bBlk + (int64_t)sp * LL, live ? LL * 4 : 0);
#pragma unroll
        for (int k = 0; k < T; ++k) {
          const int i = lane + kWave * k;
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, tile[i]), dBlk, i * 4,
                                                0, MPL_ST_AUX);
        }
      }
      st_p += ch.pstep;
    }
  }
}

template <int T>
struct PixSB {
  float a, hd, hi;
  int nidx;
  float w, de;
  float blk[T];
};

template <int T, int LT>
__global__ void __launch_bounds__(kWave) soft_bwd_kernel(const BackParams p) {
  extern __shared__ float smem[];
  const int L = LT > 0 ? LT : p.L, LL = L * L;
  const int Lp = L | 1;  // odd row stride of the transposed gradient block: conflict-free reads
  constexpr int kTile = kWave * T;
  float* tab = smem;            // LL
  float* hist = tab + LL;       // LL: per-pair dcontext accumulator [fd * L + cd]
  float* tile = hist + LL;      // kTile (>= LL): duals of the pixel, in their stored layout
  float* grad = tile + kTile;   // L * Lp: ddual[fd * Lp + cd]
  const int lane = threadIdx.x;
  const int64_t HW = (int64_t)p.H * p.W;
  const int64_t P = (int64_t)p.B * HW;
  const int64_t N = P * L;
  const ChainCtx ch = locate_chain(p);
  const int dir = ch.dir;
  const int n = ch.n;

  fill_table(p.ctx, L, p.ctx2d, lane, tab);
  for (int i = lane; i < LL; i += kWave) hist[i] = 0.f;
  __syncthreads();

  const int64_t img_p = (int64_t)ch.bv * HW;
  const int64_t img_e = img_p * L;
  const int vbytes = L * 4;
  const bool read_h = !p.first_touch;
  const float* __restrict__ bA = p.a_in + img_e;
  float* __restrict__ bAo = p.a_out + img_e;
  float* __restrict__ bHd = p.h + (int64_t)dir * N + img_e;
  float* __restrict__ bHi = p.h + (int64_t)(dir ^ 1) * N + img_e;
  const float* __restrict__ bBlk = p.edge_label + ((int64_t)dir * P + img_p) * LL;
  const int img_bytes_p = (int)(HW * 4 > 0x7fffffff ? 0x7fffffff : HW * 4);
  const rsrc_t dInorm = make_rsrc(p.idx_norm + (int64_t)dir * P + img_p, (int)HW);
  const rsrc_t dW = make_rsrc(p.edge + (int64_t)dir * P + img_p, img_bytes_p);
  // a gradient the caller does not want (null): its reads return 0 and its stores are dropped
  const rsrc_t dDe = make_rsrc(p.dedge != nullptr ? p.dedge + (int64_t)dir * P + img_p : nullptr,
                               p.dedge != nullptr ? img_bytes_p : 0);
  const float rho = p.rho;
  const int foff = lane * 4;
  const bool valid = lane < L;
  const int col = valid ? lane : L - 1;
  const bool even = (dir & 1) == 0;
  const int dstep = even ? L : 1;             // address step of the front label inside the block
  const int dbase = even ? col : col * L;     // address of (cd = lane, fd = 0)
  float tcol[LT > 0 ? LT : 1], hreg[LT > 0 ? LT : 1];  // ctx(lane, fd); dcontext partial sums
  if (LT > 0) {
#pragma unroll
    for (int fd = 0; fd < LT; ++fd) {
      tcol[fd] = tab[fd * L + col];
      hreg[fd] = 0.f;
    }
  }

  int ld_t = n - 1;
  int ld_p = ch.pix0 + (n - 1) * ch.pstep;
  auto load_next = [&]() {
    PixSB<T> r;
    const unsigned pp = (unsigned)uniform_i(ld_t >= 0 ? ld_p : ch.pix0);
    const unsigned so = pp * (unsigned)vbytes;
    const int nrec = (int)(so + (unsigned)vbytes);
    float t1[1];
    buf_load<1, true>(make_rsrc(bA, nrec), foff, so, t1);
    r.a = t1[0];
    buf_load<1, true>(make_rsrc(bHd, read_h ? nrec : 0), foff, so, t1);
    r.hd = t1[0];
    buf_load<1, true>(make_rsrc(bHi, read_h ? nrec : 0), foff, so, t1);
    r.hi = t1[0];
    r.nidx = __builtin_amdgcn_raw_buffer_load_b8(dInorm, (int)pp, 0, 0);
    r.w = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dW, (int)(pp * 4u), 0, 0));
    r.de = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dDe, (int)(pp * 4u), 0, 0));
    const rsrc_t dBlk = make_rsrc(bBlk + (int64_t)pp * LL, LL * 4);
#pragma unroll
    for (int k = 0; k < T; ++k)
      r.blk[k] = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(dBlk, (lane + kWave * k) * 4, 0, MPL_LD_AUX));
    ld_t -= 1;
    ld_p -= ch.pstep;
    return r;
  };

  constexpr int kOps = 3 + 3 + T + 3 + 1;
  constexpr int D = ring_depth(kOps);
  PixSB<T> ring[D];
#pragma unroll
  for (int u = 0; u < D; ++u) ring[u] = load_next();

  float sc = 0.f;  // dU of the current pixel: what the previous step scattered into it
  int st_p = ch.pix0 + (n - 1) * ch.pstep;
  for (int s0 = 0; s0 < n; s0 += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int t = n - 1 - (s0 + u);
      wait_vmem<(D - 1) * kOps>();
      const PixSB<T> px = ring[u];
      ring[u] = load_next();
      float scn = 0.f, det = 0.f;
      if (t >= 1) {  // the chain start (t == 0) has no incoming edge
        const float w = uniform_f(px.w);
        const int nidx = __builtin_amdgcn_readfirstlane(px.nidx);
        float gv = valid ? fmaf(rho, sc, px.a + px.hd) : 0.f;
        const float tot = wave_sum(gv);  // back norm, TRWP_backward_soft.cu:52-63
        if (lane == nidx) gv -= tot;
#pragma unroll
        for (int k = 0; k < T; ++k) tile[lane + kWave * k] = px.blk[k];
        // softmin statistics of this lane's label, :83-105
        float mn = INFINITY;
        float se = 0.f, sd = 0.f, de = 0.f;
        if constexpr (LT > 0) {
          float dual[LT], ex[LT];
#pragma unroll
          for (int fd = 0; fd < LT; ++fd) {
            dual[fd] = tile[dbase + fd * dstep];
            mn = fminf(mn, dual[fd]);
          }
#pragma unroll
          for (int fd = 0; fd < LT; ++fd) {
            ex[fd] = fast_exp(mn - dual[fd]);
            se += ex[fd];
            sd = fmaf(ex[fd], dual[fd], sd);
          }
          const float inv = 1.f / se;
          const float soft1 = fmaf(sd, inv, 1.f);
          const float gs = gv * inv;
#pragma unroll
          for (int fd = 0; fd < LT; ++fd) {
            const float dd = gs * ex[fd] * (soft1 - dual[fd]);  // :110-113
            de = fmaf(tcol[fd], dd, de);
            hreg[fd] = fmaf(w, dd, hreg[fd]);
            ex[fd] = dd;
          }
          if (valid) {  // one predicated region for the whole column, not one per store
#pragma unroll
            for (int fd = 0; fd < LT; ++fd) grad[fd * Lp + lane] = ex[fd];
          }
        } else {
#pragma unroll 4
          for (int fd = 0; fd < L; ++fd) mn = fminf(mn, tile[dbase + fd * dstep]);
#pragma unroll 4
          for (int fd = 0; fd < L; ++fd) {
            const float dual = tile[dbase + fd * dstep];
            const float e = fast_exp(mn - dual);
            se += e;
            sd = fmaf(e, dual, sd);
          }
          const float inv = 1.f / se;
          const float soft1 = fmaf(sd, inv, 1.f);
          const float gs = gv * inv;
          if (valid) {  // (lanes without a label carry gv = 0 and would add nothing)
#pragma unroll 4
            for (int fd = 0; fd < L; ++fd) {
              const float dual = tile[dbase + fd * dstep];
              const float dd = gs * fast_exp(mn - dual) * (soft1 - dual);  // :110-113
              de = fmaf(tab[fd * L + col], dd, de);
              hist[fd * L + lane] = fmaf(w, dd, hist[fd * L + lane]);  // this lane's own entries
              grad[fd * Lp + lane] = dd;
            }
          }
        }
        // dU[q, fd] = sum_cd ddual[cd, fd]: lane fd adds up its row of the transposed block
        if (valid) {
#pragma unroll 4
          for (int cd = 0; cd < L; ++cd) scn += grad[lane * Lp + cd];
        }
        det = wave_sum(de);
      }
      const unsigned sp = (unsigned)uniform_i(st_p);
      const unsigned so = sp * (unsigned)vbytes;
      const int nrec = t >= 0 ? (int)(so + (unsigned)vbytes) : 0;
      const float an = fmaf(rho, sc, px.a);  // g_k += rho*dU for every k, dunary too
      const float a1[1] = {an}, h1[1] = {-an}, i1[1] = {px.hi - sc};
      buf_store<1, true>(make_rsrc(bAo, nrec), foff, so, a1);
      buf_store<1, true>(make_rsrc(bHd, nrec), foff, so, h1);
      buf_store<1, true>(make_rsrc(bHi, nrec), foff, so, i1);
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, px.de + det), dDe,
                                            t >= 1 ? (int)(sp * 4u) : kDeadOffset, 0, 0);
      sc = scn;
      st_p -= ch.pstep;
    }
  }
  if (p.dctx == nullptr) return;
  if (LT > 0 && valid) {
#pragma unroll
    for (int fd = 0; fd < LT; ++fd) hist[fd * L + lane] = hreg[fd];
  }
  __syncthreads();
  // fold the pair table into dcontext's bins: |cd - fd| (1-D) or [min, max] (2-D), the diagonal
  // included (TRWP_backward_soft.cu:116-126)
  if (!p.ctx2d) {
    if (valid) {
      float acc = 0.f;
      for (int fd = 0; fd < L; ++fd) {
        if (fd + lane < L) acc += hist[fd * L + fd + lane];
        if (lane > 0 && fd - lane >= 0) acc += hist[fd * L + fd - lane];
      }
      if (acc != 0.f) atomicAdd(&p.dctx[lane], acc);
    }
  } else {
    for (int i = lane; i < LL; i += kWave) {
      const int fd = i / L, cd = i - fd * L;
      if (cd > fd) continue;  // handled by the (fd, cd) entry
      const float v = hist[i] + (cd < fd ? hist[cd * L + fd] : 0.f);
      if (v != 0.f) atomicAdd(&p.dctx[cd * L + fd], v);
    }
  }
}

// Stand-alone softmin of stored blocks (SoftWeightedMessageKernel / ...BackKernel,
// TRWP_hard_soft/TRWP_swbp.cu:131-254): message (n_trees, L, L) laid out [fd][cd];
//   out[tree, cd] = sum_fd prob * message - min_cd(...),  prob = softmax_fd(-message[:, cd])
// One wavefront per tree, lane i owns labels i, i + 64, ... (consecutive lanes read consecutive
// floats of a row).
constexpr int kSwmR = kMaxL / kWave;

__device__ __forceinline__ void swm_stats(const float* __restrict__ blk, int L, int lane,
                                          float (&mn)[kSwmR], float (&inv)[kSwmR],
                                          float (&soft)[kSwmR]) {
#pragma unroll
  for (int j = 0; j < kSwmR; ++j) {
    const int cd = lane + kWave * j;
    mn[j] = INFINITY;
    inv[j] = 0.f;
    soft[j] = 0.f;
    if (cd < L) {
      for (int fd = 0; fd < L; ++fd) mn[j] = fminf(mn[j], blk[fd * L + cd]);
      float se = 0.f, sd = 0.f;
      for (int fd = 0; fd < L; ++fd) {
        const float v = blk[fd * L + cd];
        const float e = expf(-(v - mn[j]));
        se += e;
        sd = fmaf(e, v, sd);
      }
      inv[j] = 1.f / se;
      soft[j] = sd * inv[j];
    }
  }
}

__global__ void __launch_bounds__(kWave) swm_fwd_kernel(const float* __restrict__ msg, int n_trees,
                                                        int L, float* __restrict__ out,
                                                        uint8_t* __restrict__ min_ind) {
  const int lane = threadIdx.x;
  for (int tree = blockIdx.x; tree < n_trees; tree += gridDim.x) {
    float mn[kSwmR], inv[kSwmR], soft[kSwmR];
    swm_stats(msg + (int64_t)tree * L * L, L, lane, mn, inv, soft);
    float lo = INFINITY;
#pragma unroll
    for (int j = 0; j < kSwmR; ++j) lo = fminf(lo, (lane + kWave * j < L) ? soft[j] : INFINITY);
    const float nmin = wave_min(lo);
    int arg = -1;  // largest label that attains the minimum (TRWP_swbp.cu:95-101)
#pragma unroll
    for (int j = 0; j < kSwmR; ++j) {
      const int cd = lane + kWave * j;
      if (cd < L) {
        out[(int64_t)tree * L + cd] = soft[j] - nmin;
        if (soft[j] == nmin) arg = cd;
      }
    }
    const float best = -wave_min(-(float)arg);
    if (lane == 0) min_ind[tree] = (uint8_t)(int)best;
  }
}

__global__ void __launch_bounds__(kWave) swm_bwd_kernel(const float* __restrict__ dout,
                                                        const float* __restrict__ msg,
                                                        const uint8_t* __restrict__ min_ind,
                                                        int n_trees, int L,
                                                        float* __restrict__ dmsg) {
  const int lane = threadIdx.x;
  for (int tree = blockIdx.x; tree < n_trees; tree += gridDim.x) {
    const float* blk = msg + (int64_t)tree * L * L;
    float mn[kSwmR], inv[kSwmR], soft[kSwmR], g[kSwmR];
    swm_stats(blk, L, lane, mn, inv, soft);
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < kSwmR; ++j) {
      const int cd = lane + kWave * j;
      g[j] = cd < L ? dout[(int64_t)tree * L + cd] : 0.f;
      part += g[j];
    }
    const float tot = wave_sum(part);
    const int ind = min_ind[tree];
#pragma unroll
    for (int j = 0; j < kSwmR; ++j) {
      const int cd = lane + kWave * j;
      if (cd == ind) g[j] -= tot;
      if (cd < L) {
        for (int fd = 0; fd < L; ++fd) {
          const float v = blk[fd * L + cd];
          const float prob = expf(-(v - mn[j])) * inv[j];
          dmsg[(int64_t)tree * L * L + fd * L + cd] = g[j] * prob * (1.f - v + soft[j]);
        }
      }
    }
  }
}

int tile_bucket(int L) {
  const int need = (L * L + kWave - 1) / kWave;
  return need <= 4 ? 4 : (need <= 7 ? 7 : (need <= 16 ? 16 : 64));
}

}  // namespace

void launch_soft_fwd(const SweepParams& p, bool train, hipStream_t st) {
  const int blocks = p.block_prefix[p.n_dirs];
  if (blocks <= 0) return;
  const int LL = p.L * p.L;
  const int T = tile_bucket(p.L);
  const size_t lds = sizeof(float) * (LL + (train ? (LL > kWave * T ? LL : kWave * T) : 0));
  if (!train) {
    if (p.L == 21)
      soft_fwd_kernel<false, 0, 21><<<blocks, kWave, lds, st>>>(p);
    else
      soft_fwd_kernel<false, 0, 0><<<blocks, kWave, lds, st>>>(p);
    return;
  }
  if (p.L == 21) {
    soft_fwd_kernel<true, 7, 21><<<blocks, kWave, lds, st>>>(p);
    return;
  }
  switch (T) {
    case 4: soft_fwd_kernel<true, 4, 0><<<blocks, kWave, lds, st>>>(p); break;
    case 7: soft_fwd_kernel<true, 7, 0><<<blocks, kWave, lds, st>>>(p); break;
    case 16: soft_fwd_kernel<true, 16, 0><<<blocks, kWave, lds, st>>>(p); break;
    default: soft_fwd_kernel<true, 64, 0><<<blocks, kWave, lds, st>>>(p); break;
  }
}

void launch_soft_bwd(const BackParams& p, hipStream_t st) {
  const int blocks = p.block_prefix[p.n_dirs];
  if (blocks <= 0) return;
  const int LL = p.L * p.L;
  const int T = tile_bucket(p.L);
  const size_t lds = sizeof(float) * (2 * LL + kWave * T + p.L * (p.L | 1));
  if (p.L == 21) {
    soft_bwd_kernel<7, 21><<<blocks, kWave, lds, st>>>(p);
    return;
  }
  switch (T) {
    case 4: soft_bwd_kernel<4, 0><<<blocks, kWave, lds, st>>>(p); break;
    case 7: soft_bwd_kernel<7, 0><<<blocks, kWave, lds, st>>>(p); break;
    case 16: soft_bwd_kernel<16, 0><<<blocks, kWave, lds, st>>>(p); break;
    default:
      // up to 66 KB of LDS at 64 labels: above the default limit of a workgroup
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&soft_bwd_kernel<64, 0>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      soft_bwd_kernel<64, 0><<<blocks, kWave, lds, st>>>(p);
      break;
  }
}

void launch_swm_fwd(const float* msg, int n_trees, int L, float* out, uint8_t* min_ind,
                    hipStream_t st) {
  if (n_trees <= 0) return;
  swm_fwd_kernel<<<n_trees < 65536 ? n_trees : 65536, kWave, 0, st>>>(msg, n_trees, L, out, min_ind);
}

void launch_swm_bwd(const float* dout, const float* msg, const uint8_t* min_ind, int n_trees, int L,
                    float* dmsg, hipStream_t st) {
  if (n_trees <= 0) return;
  swm_bwd_kernel<<<n_trees < 65536 ? n_trees : 65536, kWave, 0, st>>>(dout, msg, min_ind, n_trees, L,
                                                                     dmsg);
}

}  // namespace mpl
