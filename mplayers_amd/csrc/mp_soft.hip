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
// Mapping (up to 64 labels; the kernels for more are further down): one wavefront per chain, one
// label per lane, pixel planes prefetched through a register ring as in the hard kernels.  The (L, L) block goes through LDS so that global memory
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

// One label per lane: 33 to 64 labels; fewer labels take the lane-split kernels below, more the
// several-labels-per-lane ones.
template <bool TRAIN, int T>
__global__ void __launch_bounds__(kWave) soft_fwd_kernel(const SweepParams p) {
  extern __shared__ float smem[];
  const int L = p.L, LL = L * L;
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
    __builtin_amdgcn_sched_barrier(0);  // (the chain start's loads stay ahead of the ring's)
    const float un = fmaf(p0.s - p0.md, rho, -p0.mi);
    uf = valid ? un : inf;
  }

  constexpr int kOps = 4 + 2 + (TRAIN ? 1 + T : 0);
  constexpr int D = ring_depth(kOps);
  PixSF ring[D], ring2[D];  // two banks, filled and used in turn: no register is moved
#pragma unroll
  for (int u = 0; u < D; ++u) {
    ring[u] = load_next();
    // keeps the pixels' loads in this order: the compiler's own waits in the loop are sized for
    // the order it sees here, and a later pixel's loads placed first would make them drain the queue
    __builtin_amdgcn_sched_barrier(0);
  }

  int st_p = ch.pix0 + ch.pstep;
  auto step = [&](const PixSF& px, const int t) __attribute__((always_inline)) {
      const bool live = t < n;
      const float tt = px.s - px.md;
      const float un = valid ? fmaf(tt, rho, -px.mi) : inf;  // UpdateUnaryKernelSoft, :161-181
      const float w = uniform_f(px.w);
      const float a = fmaf(rho, prev, uf);  // lane = front label
      // pass 1: minimum of the duals of this lane's label; the block goes to LDS
      float mn = inf;
      float se = 0.f, sd = 0.f;
#pragma unroll 4
      for (int fd = 0; fd < L; ++fd) {
        const float dual = fmaf(w, tab[fd * L + col], readlane_f(a, fd));
        mn = fminf(mn, dual);
        if (TRAIN && valid) tile[wbase + fd * wstep] = dual;
      }
      // pass 2: softmin weights and the expected dual
#pragma unroll 4
      for (int fd = 0; fd < L; ++fd) {
        const float dual = fmaf(w, tab[fd * L + col], readlane_f(a, fd));
        const float e = fast_exp(mn - dual);
        se += e;
        sd = fmaf(e, dual, sd);
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
  };
  for (int t0 = 1; t0 < n; t0 += 2 * D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      // the loads of this ring slot were followed by at most D-1 steps' worth of memory operations
      wait_vmem<(D - 1) * kOps>();
      const auto px = ring[u];
      ring2[u] = load_next();
      __builtin_amdgcn_sched_barrier(0);  // the next pixel's loads go out before this step's work
      step(px, t0 + u);
    }
    if (t0 + D >= n) break;  // wave-uniform
#pragma unroll
    for (int u = 0; u < D; ++u) {
      wait_vmem<(D - 1) * kOps>();
      const auto px = ring2[u];
      ring[u] = load_next();
      __builtin_amdgcn_sched_barrier(0);
      step(px, t0 + D + u);
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

template <int T>
__global__ void __launch_bounds__(kWave) soft_bwd_kernel(const BackParams p) {
  extern __shared__ float smem[];
  const int L = p.L, LL = L * L;
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
  PixSB<T> ring[D], ring2[D];  // two banks, filled and used in turn: no register is moved
#pragma unroll
  for (int u = 0; u < D; ++u) {
    ring[u] = load_next();
    // keeps the pixels' loads in this order: the compiler's own waits in the loop are sized for
    // the order it sees here, and a later pixel's loads placed first would make them drain the queue
    __builtin_amdgcn_sched_barrier(0);
  }

  float sc = 0.f;  // dU of the current pixel: what the previous step scattered into it
  int st_p = ch.pix0 + (n - 1) * ch.pstep;
  auto step = [&](const PixSB<T>& px, const int t) __attribute__((always_inline)) {
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
  };
  for (int s0 = 0; s0 < n; s0 += 2 * D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      // the loads of this ring slot were followed by at most D-1 steps' worth of memory operations
      wait_vmem<(D - 1) * kOps>();
      const auto px = ring[u];
      ring2[u] = load_next();
      __builtin_amdgcn_sched_barrier(0);  // the next pixel's loads go out before this step's work
      step(px, n - 1 - (s0 + u));
    }
    if (s0 + D >= n) break;  // wave-uniform
#pragma unroll
    for (int u = 0; u < D; ++u) {
      wait_vmem<(D - 1) * kOps>();
      const auto px = ring2[u];
      ring[u] = load_next();
      __builtin_amdgcn_sched_barrier(0);
      step(px, n - 1 - (s0 + D + u));
    }
  }
  if (p.dctx == nullptr) return;
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

// ------------------------------------------------------------------------------------------------
// At most 32 labels: with one label per lane a third or less of the wavefront works, and the step
// is L exponentials per lane deep.  Here the front labels of the chain's pixel are split over
// G = 4 / 3 / 2 groups of lanes (L <= 16 / 21 / 32): lane g * L + cd carries label cd like its
// G - 1 replicas in the other groups (they load the same values and keep the same recurrence
// state) but only looks at the front labels g * F .. g * F + F - 1, F = ceil(L / G).  Each lane
// forms the softmin statistics of its F duals around their own minimum; one exchange
// (ds_bpermute: every lane fetches the G partial triples of its label and combines them in group
// order, so the replicas stay bit-identical) rescales them to the minimum over all front labels.
// The duals move between registers and memory directly, F dwords per lane at the lane's places of
// the pixel's block; the lanes of group 0 store the label vectors.  FM: compile-time bound of F.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float bperm_f(int addr, float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(addr, __builtin_bit_cast(int, x)));
}
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
constexpr float kLog2e = 1.4426950408889634f;
// exp(m - x) with m * kLog2e given: one multiply-add and the hardware's 2^x
__device__ __forceinline__ float exp_below(float x, float m_log2e) {
  return __builtin_amdgcn_exp2f(fmaf(x, -kLog2e, m_log2e));
}

// Reductions as chains of DPP-fused operations (a lane without a source lane keeps its value; a
// DPP operand written by the instruction before needs two wait states, which the compiler cannot
// see inside a statement: each instruction carries its own, and a chain is one statement, since
// the compiler pads the gap between two statements itself).  NL = 16 / 32 / 64: over the first NL
// lanes only, the others are ignored; the result is wave-uniform.
#define MPL_RED_DPP(OP, CTRL) "s_nop 1\n\t" OP " %0, %0, %0 " CTRL " bank_mask:0xf\n\t"
#define MPL_RED_ROW(OP)                                                            \
  MPL_RED_DPP(OP, "row_shr:1 row_mask:0xf") MPL_RED_DPP(OP, "row_shr:2 row_mask:0xf") \
      MPL_RED_DPP(OP, "row_shr:4 row_mask:0xf") MPL_RED_DPP(OP, "row_shr:8 row_mask:0xf")
#define MPL_RED_LANES(OP)                                                                      \
  if constexpr (NL <= 16)                                                                      \
    asm(MPL_RED_ROW(OP) "s_nop 0" : "+v"(x));                                                  \
  else if constexpr (NL <= 32)                                                                 \
    asm(MPL_RED_ROW(OP) MPL_RED_DPP(OP, "row_bcast:15 row_mask:0xa") "s_nop 0" : "+v"(x));     \
  else                                                                                         \
    asm(MPL_RED_ROW(OP) MPL_RED_DPP(OP, "row_bcast:15 row_mask:0xa")                           \
            MPL_RED_DPP(OP, "row_bcast:31 row_mask:0xc") "s_nop 0"                             \
        : "+v"(x))
template <int NL>
__device__ __forceinline__ float lanes_sum(float x) {
  MPL_RED_LANES("v_add_f32_dpp");
  return readlane_f(x, NL - 1);
}
template <int NL>
__device__ __forceinline__ float lanes_min(float x) {
  MPL_RED_LANES("v_min_f32_dpp");
  return readlane_f(x, NL - 1);
}
#undef MPL_RED_LANES
#undef MPL_RED_ROW
#undef MPL_RED_DPP

// (minimum, sum of weights, weighted sum of duals) of a label over all its front labels from the
// per-lane partial triples, each taken around its own minimum.  `scale` returns the factor that
// turns this lane's weights exp(mn_lane - dual) into exp(mn - dual).
template <int G>
__device__ __forceinline__ void group_softmin(const int (&addr)[G], float mn_l, float se_l,
                                              float sd_l, float& mn, float& se, float& sd,
                                              float& scale) {
  float pm[G], ps[G], pd[G];
#pragma unroll
  for (int k = 0; k < G; ++k) {
    pm[k] = bperm_f(addr[k], mn_l);
    ps[k] = bperm_f(addr[k], se_l);
    pd[k] = bperm_f(addr[k], sd_l);
  }
  mn = pm[0];
#pragma unroll
  for (int k = 1; k < G; ++k) mn = fminf(mn, pm[k]);
  se = 0.f;
  sd = 0.f;
#pragma unroll
  for (int k = 0; k < G; ++k) {
    const float f = exp_below(pm[k], mn * kLog2e);  // (a group without front labels: 2^-inf = 0)
    se = fmaf(f, ps[k], se);
    sd = fmaf(f, pd[k], sd);
  }
  scale = exp_below(mn_l, mn * kLog2e);
}

template <int FM>
struct PixSS {
  float a, hd, hi, w, de;
  int nidx;
  float dual[FM];
};

// NT4: float4 stores per lane that cover the pixel's block of duals (256 * NT4 >= L * L)
template <bool TRAIN, int G, int FM, int NT4>
__global__ void __launch_bounds__(kWave) soft_split_fwd_kernel(const SweepParams p) {
  extern __shared__ float smem[];
  const int L = p.L, LL = L * L;
  float* tile = smem;              // 256 * NT4 floats (training): the pixel's block as it is stored
  float* tab = smem + (TRAIN ? 256 * NT4 : 0);  // LL floats (training: and a spare word per lane)
  const int lane = threadIdx.x;
  const ChainCtx ch0 = locate_chain(p);
  if (ch0.n < 2) return;  // nothing to write
  fill_table(p.ctx, L, p.ctx2d, lane, tab);
  __syncthreads();

  // chain-starved launches (p.fused_pair): the wavefront sweeps its chain for dirs[0] and then, over
  // the same pixels in reverse, for the opposite direction, reading back what it stored
  const int halves = p.fused_pair ? 2 : 1;
#pragma clang loop unroll(disable)
  for (int half = 0; half < halves; ++half) {
  ChainCtx ch = ch0;
  if (half) {
    ch.dir = ch0.dir ^ 1;
    ch.pix0 = ch0.pix0 + (ch0.n - 1) * ch0.pstep;
    ch.pstep = -ch0.pstep;
    wait_vmem<0>();
    __syncthreads();
  }
  const int64_t HW = (int64_t)p.H * p.W;
  const int64_t P = (int64_t)p.B * HW;
  const int64_t N = P * L;
  const int dir = ch.dir;
  const int64_t img_p = (int64_t)ch.bv * HW;
  const int64_t img_e = img_p * L;
  const int vbytes = L * 4;
  // one descriptor per plane over the batch item's image; a lane without work carries an offset
  // that no descriptor covers
  const int img_bytes = (int)(unsigned)(HW * L * 4);
  const rsrc_t rS = make_rsrc(p.belief + img_e, img_bytes);
  const rsrc_t rMd = make_rsrc(p.msg_in + (int64_t)dir * N + img_e, img_bytes);
  const rsrc_t rMi = make_rsrc(p.msg_in + (int64_t)(dir ^ 1) * N + img_e, img_bytes);
  const rsrc_t rMo = make_rsrc(p.msg_out + (int64_t)dir * N + img_e, img_bytes);
  const rsrc_t rSo = make_rsrc(p.belief_out + img_e, img_bytes);
  float* __restrict__ bBlk = TRAIN ? p.edge_label + ((int64_t)dir * P + img_p) * LL : nullptr;
  const int img_bytes_p = (int)(HW * 4 > 0x7fffffff ? 0x7fffffff : HW * 4);
  const rsrc_t dW = make_rsrc(p.edge + (int64_t)dir * P + img_p, img_bytes_p);
  const rsrc_t dInorm = make_rsrc(TRAIN ? p.idx_norm + (int64_t)dir * P + img_p : nullptr,
                                  TRAIN ? (int)HW : 0);
  const float rho = p.rho;
  const float inf = INFINITY;
  const int n = ch.n;
  const int F = (L + G - 1) / G;
  const bool valid = lane < G * L;
  const int g = valid ? lane / L : 0;
  const int cd = valid ? lane - g * L : 0;
  const bool store_lane = lane < L;  // group 0
  const unsigned foff = (unsigned)cd * 4u;
  const bool even = (dir & 1) == 0;
  int addr[G];
#pragma unroll
  for (int k = 0; k < G; ++k) addr[k] = (valid ? k * L + cd : lane) * 4;
  // this lane's front labels fd0 + i; beyond the last label the entry repeats it with weight 0
  const int fd0 = g * F;
  float tcol[FM];
  int src[FM], tidx[FM];
  bool inr[FM];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    inr[i] = valid && i < F && fd0 + i < L;
    const int fd = inr[i] ? fd0 + i : L - 1;
    tcol[i] = tab[fd * L + cd];  // ctx(cd, fd)
    src[i] = fd * 4;             // a[fd] from group 0's replica
    // place of (cd, fd) inside the stored block; an entry that does not exist goes to a spare word
    // of this lane behind the table (a store to somewhere costs one instruction, a skipped one a
    // save, a branch and a restore of the execution mask)
    tidx[i] = inr[i] ? (even ? fd * L + cd : cd * L + fd) : 256 * NT4 + LL + lane;
  }
  // the block leaves as NT4 16-byte stores per lane and, L * L being 0 or 1 modulo 4, one last dword
  int qoff[NT4];
#pragma unroll
  for (int k = 0; k < NT4; ++k) {
    const int q = lane + kWave * k;
    qoff[k] = 4 * q + 3 < LL ? 16 * q : kDeadOffset;
  }
  const int tail_off = (lane == 0 && (LL & 3)) ? (LL - 1) * 4 : kDeadOffset;

  const int last_p = ch.pix0 + (n - 1) * ch.pstep;
  int ld_p = ch.pix0;
  int ld_t = 0;
  auto load_next = [&]() __attribute__((always_inline)) {
    PixSF r;
    const unsigned pp = (unsigned)uniform_i(ld_t < n ? ld_p : last_p);
    const int vo = (int)(valid ? pp * (unsigned)vbytes + foff : kDeadWide);
    float t1[1];
    buf_load<1, true>(rS, vo, 0u, t1);
    r.s = t1[0];
    buf_load<1, true>(rMd, vo, 0u, t1);
    r.md = t1[0];
    buf_load<1, true>(rMi, vo, 0u, t1);
    r.mi = t1[0];
    r.w = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dW, (int)(pp * 4u), 0, 0));
    ld_p += ch.pstep;
    ld_t += 1;
    return r;
  };

  float prev = 0.f, uf;
  {
    const PixSF p0 = load_next();
    __builtin_amdgcn_sched_barrier(0);  // (the chain start's loads stay ahead of the ring's)
    uf = fmaf(p0.s - p0.md, rho, -p0.mi);
  }

  constexpr int kOps = 4 + 2 + (TRAIN ? 2 + NT4 : 0);
  constexpr int D = ring_depth(kOps);
  PixSF ring[D], ring2[D];  // two banks, filled and used in turn: no register is moved
#pragma unroll
  for (int u = 0; u < D; ++u) {
    ring[u] = load_next();
    // keeps the pixels' loads in this order: the compiler's own waits in the loop are sized for
    // the order it sees here, and a later pixel's loads placed first would make them drain the queue
    __builtin_amdgcn_sched_barrier(0);
  }

  int st_p = ch.pix0 + ch.pstep;
  auto step = [&](const PixSF& px, const int t) __attribute__((always_inline)) {
      const bool live = t < n;
      const float tt = px.s - px.md;
      const float un = fmaf(tt, rho, -px.mi);  // UpdateUnaryKernelSoft, TRWP_forward_soft.cu:161-181
      const float w = uniform_f(px.w);
      const float a = fmaf(rho, prev, uf);  // (every group holds the same a)
      // this lane's duals and their softmin statistics around their own minimum (:81-97)
      float dual[FM];
      float mn_l = inf;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        dual[i] = fmaf(w, tcol[i], bperm_f(src[i], a));
        mn_l = fminf(mn_l, inr[i] ? dual[i] : inf);
      }
      float se_l = 0.f, sd_l = 0.f;
      const float ml2 = mn_l * kLog2e;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const float e = inr[i] ? exp_below(dual[i], ml2) : 0.f;
        se_l += e;
        sd_l = fmaf(e, dual[i], sd_l);
      }
      if (TRAIN) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
          tile[tidx[i]] = dual[i];
      }
      float mn, se, sd, scale;
      group_softmin<G>(addr, mn_l, se_l, sd_l, mn, se, sd, scale);
      const float soft = sd * fast_rcp(se);
      const float nmin = lanes_min<(G == 4 ? 16 : 32)>(store_lane ? soft : inf);
      const float m = soft - nmin;
      prev = m;
      uf = un;
      const unsigned sp = (unsigned)uniform_i(st_p);
      const int vo = (int)((store_lane && live) ? sp * (unsigned)vbytes + foff : kDeadWide);
      const float m1[1] = {m}, s1[1] = {tt + m};
      buf_store<1, true>(rMo, vo, 0u, m1);
      buf_store<1, true>(rSo, vo, 0u, s1);
      if (TRAIN) {
        const bool pr[1] = {store_lane && (soft == nmin)};
        const int nidx = last_label<1>(pr, L - 1);
        __builtin_amdgcn_raw_buffer_store_b8((unsigned char)nidx, dInorm,
                                             live ? (int)sp : kDeadOffset, 0, 0);
        const rsrc_t dBlk = make_rsrc(bBlk + (int64_t)sp * LL, live ? LL * 4 : 0);
#pragma unroll
        for (int k = 0; k < NT4; ++k) {
          const float4 v = reinterpret_cast<const float4*>(tile)[lane + kWave * k];
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), dBlk, qoff[k], 0,
                                                 MPL_ST_AUX);
        }
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, tile[LL - 1]), dBlk,
                                              tail_off, 0, MPL_ST_AUX);
      }
      st_p += ch.pstep;
  };
  for (int t0 = 1; t0 < n; t0 += 2 * D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      // the loads of this ring slot were followed by at most D-1 steps' worth of memory operations
      wait_vmem<(D - 1) * kOps>();
      const auto px = ring[u];
      ring2[u] = load_next();
      __builtin_amdgcn_sched_barrier(0);  // the next pixel's loads go out before this step's work
      step(px, t0 + u);
    }
    if (t0 + D >= n) break;  // wave-uniform
#pragma unroll
    for (int u = 0; u < D; ++u) {
      wait_vmem<(D - 1) * kOps>();
      const auto px = ring2[u];
      ring[u] = load_next();
      __builtin_amdgcn_sched_barrier(0);
      step(px, t0 + D + u);
    }
  }
  }  // both sweeps of a fused pair
}

// NQ: float4 reads that cover a row of the gradient block (4 * NQ >= L).  The duals come straight
// from memory into the registers of the lanes that use them (F gathers per lane: staging the block
// through LDS with 16-byte loads, as the forward scan stores it, measured slower here).
template <int G, int FM, int NQ>
__global__ void __launch_bounds__(kWave) soft_split_bwd_kernel(const BackParams p) {
  extern __shared__ float smem[];
  const int L = p.L, LL = L * L;
  constexpr int S = 4 * NQ;  // row stride of the gradient block
  float* tab = smem;         // LL
  const int LLp = (LL + 3) & ~3;  // (keeps the rows of the gradient block 16-byte aligned)
  float* hist = tab + LLp;   // LL: per-pair dcontext accumulator [fd * L + cd]
  float* grad = hist + LLp;  // L rows of S: ddual[fd * S + cd], 0 beyond cd = L - 1; a spare word per lane
  const int lane = threadIdx.x;
  const int64_t HW = (int64_t)p.H * p.W;
  const int64_t P = (int64_t)p.B * HW;
  const int64_t N = P * L;
  const ChainCtx ch0 = locate_chain(p);
  const int n = ch0.n;

  fill_table(p.ctx, L, p.ctx2d, lane, tab);
  for (int i = lane; i < LL; i += kWave) hist[i] = 0.f;
  for (int i = lane; i < L * S; i += kWave) grad[i] = 0.f;
  __syncthreads();

  float hreg[FM];  // dcontext partial sums of this lane's (cd, fd) pairs, over both walks of a pair
#pragma unroll
  for (int i = 0; i < FM; ++i) hreg[i] = 0.f;
  // chain-starved launches (p.fused_pair): the odd direction's walk, then the even one's over the
  // same pixels in reverse
  const int halves = p.fused_pair ? 2 : 1;
#pragma clang loop unroll(disable)
  for (int half = 0; half < halves; ++half) {
  ChainCtx ch = ch0;
  bool first_touch = p.first_touch != 0;
  const float* a_in = p.a_in;
  if (half) {
    ch.dir = ch0.dir ^ 1;
    ch.pix0 = ch0.pix0 + (n - 1) * ch0.pstep;
    ch.pstep = -ch0.pstep;
    first_touch = false;
    a_in = p.a_out;
    wait_vmem<0>();
    __syncthreads();
  }
  const int dir = ch.dir;
  const int64_t img_p = (int64_t)ch.bv * HW;
  const int64_t img_e = img_p * L;
  const int vbytes = L * 4;
  const bool read_h = !first_touch;
  const int img_bytes = (int)(unsigned)(HW * L * 4);
  const rsrc_t rA = make_rsrc(a_in + img_e, img_bytes);
  const rsrc_t rAo = make_rsrc(p.a_out + img_e, img_bytes);
  float* const bHd = p.h + (int64_t)dir * N + img_e;
  float* const bHi = p.h + (int64_t)(dir ^ 1) * N + img_e;
  const rsrc_t rHdIn = make_rsrc(bHd, read_h ? img_bytes : 0);
  const rsrc_t rHiIn = make_rsrc(bHi, read_h ? img_bytes : 0);
  const rsrc_t rHd = make_rsrc(bHd, img_bytes);
  const rsrc_t rHi = make_rsrc(bHi, img_bytes);
  const float* __restrict__ bBlk = p.edge_label + ((int64_t)dir * P + img_p) * LL;
  const int img_bytes_p = (int)(HW * 4 > 0x7fffffff ? 0x7fffffff : HW * 4);
  const rsrc_t dInorm = make_rsrc(p.idx_norm + (int64_t)dir * P + img_p, (int)HW);
  const rsrc_t dW = make_rsrc(p.edge + (int64_t)dir * P + img_p, img_bytes_p);
  const rsrc_t dDe = make_rsrc(p.dedge != nullptr ? p.dedge + (int64_t)dir * P + img_p : nullptr,
                               p.dedge != nullptr ? img_bytes_p : 0);
  const float rho = p.rho;
  const float inf = INFINITY;
  const int F = (L + G - 1) / G;
  const bool valid = lane < G * L;
  const int g = valid ? lane / L : 0;
  const int cd = valid ? lane - g * L : 0;
  const bool store_lane = lane < L;
  const unsigned foff = (unsigned)cd * 4u;
  const bool even = (dir & 1) == 0;
  int addr[G];
#pragma unroll
  for (int k = 0; k < G; ++k) addr[k] = (valid ? k * L + cd : lane) * 4;
  const int fd0 = g * F;
  float tcol[FM];
  int boff[FM], gidx[FM];
  bool inr[FM];
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    inr[i] = valid && i < F && fd0 + i < L;
    const int fd = inr[i] ? fd0 + i : L - 1;
    tcol[i] = tab[fd * L + cd];
    // place of (cd, fd) inside the pixel's stored block
    boff[i] = inr[i] ? (even ? fd * L + cd : cd * L + fd) * 4 : kDeadOffset;
    gidx[i] = inr[i] ? fd * S + cd : L * S + lane;  // (a spare word per lane behind the block)
  }
  const float4* grow = reinterpret_cast<const float4*>(grad + cd * S);  // row of front label cd

  int ld_t = n - 1;
  int ld_p = ch.pix0 + (n - 1) * ch.pstep;
  auto load_next = [&]() __attribute__((always_inline)) {
    PixSS<FM> r;
    const unsigned pp = (unsigned)uniform_i(ld_t >= 0 ? ld_p : ch.pix0);
    const int vo = (int)(valid ? pp * (unsigned)vbytes + foff : kDeadWide);
    float t1[1];
    buf_load<1, true>(rA, vo, 0u, t1);
    r.a = t1[0];
    buf_load<1, true>(rHdIn, vo, 0u, t1);
    r.hd = t1[0];
    buf_load<1, true>(rHiIn, vo, 0u, t1);
    r.hi = t1[0];
    r.nidx = __builtin_amdgcn_raw_buffer_load_b8(dInorm, (int)pp, 0, 0);
    r.w = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dW, (int)(pp * 4u), 0, 0));
    r.de = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dDe, (int)(pp * 4u), 0, 0));
    const rsrc_t dBlk = make_rsrc(bBlk + (int64_t)pp * LL, LL * 4);
#pragma unroll
    for (int i = 0; i < FM; ++i)
      r.dual[i] = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(dBlk, boff[i], 0, MPL_LD_AUX));
    ld_t -= 1;
    ld_p -= ch.pstep;
    return r;
  };

  constexpr int kOps = 3 + 3 + FM + 3 + 1;
  constexpr int D = ring_depth(kOps);
  PixSS<FM> ring[D], ring2[D];  // two banks, filled and used in turn: no register is moved
#pragma unroll
  for (int u = 0; u < D; ++u) {
    ring[u] = load_next();
    // keeps the pixels' loads in this order: the compiler's own waits in the loop are sized for
    // the order it sees here, and a later pixel's loads placed first would make them drain the queue
    __builtin_amdgcn_sched_barrier(0);
  }

  float sc = 0.f;  // dU of the current pixel (every group holds the same value)
  int st_p = ch.pix0 + (n - 1) * ch.pstep;
  auto step = [&](const PixSS<FM>& px, const int t) __attribute__((always_inline)) {
      float scn = 0.f, det = 0.f;
      if (t >= 1) {  // the chain start (t == 0) has no incoming edge
        const float w = uniform_f(px.w);
        const int nidx = __builtin_amdgcn_readfirstlane(px.nidx);
        float gv = valid ? fmaf(rho, sc, px.a + px.hd) : 0.f;
        // back norm, TRWP_backward_soft.cu:52-63
        const float tot = lanes_sum<(G == 4 ? 16 : 32)>(store_lane ? gv : 0.f);
        if (cd == nidx) gv -= tot;
        // softmin statistics of this lane's label over all its front labels (:83-105)
        float ex[FM];
        float mn_l = inf;
#pragma unroll
        for (int i = 0; i < FM; ++i) mn_l = fminf(mn_l, inr[i] ? px.dual[i] : inf);
        float se_l = 0.f, sd_l = 0.f;
        const float ml2 = mn_l * kLog2e;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          ex[i] = inr[i] ? exp_below(px.dual[i], ml2) : 0.f;
          se_l += ex[i];
          sd_l = fmaf(ex[i], px.dual[i], sd_l);
        }
        float mn, se, sd, scale;
        group_softmin<G>(addr, mn_l, se_l, sd_l, mn, se, sd, scale);
        const float inv = fast_rcp(se);
        const float soft1 = fmaf(sd, inv, 1.f);
        const float gs = gv * inv * scale;
        float de = 0.f;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          // :110-113; nothing beyond the last label, and nothing on an idle lane (whose se is 0)
          const float dd = inr[i] ? gs * ex[i] * (soft1 - px.dual[i]) : 0.f;
          de = fmaf(tcol[i], dd, de);
          hreg[i] = fmaf(w, dd, hreg[i]);
          grad[gidx[i]] = dd;
        }
        // dU[q, fd] = sum_cd ddual[cd, fd]: every lane of label fd adds up the row in the same order
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const float4 v = grow[q];
          scn += (v.x + v.y) + (v.z + v.w);
        }
        det = lanes_sum<kWave>(de);
      }
      const unsigned sp = (unsigned)uniform_i(st_p);
      const int vo = (int)((store_lane && t >= 0) ? sp * (unsigned)vbytes + foff : kDeadWide);
      const float an = fmaf(rho, sc, px.a);  // g_k += rho*dU for every k, dunary too
      const float a1[1] = {an}, h1[1] = {-an}, i1[1] = {px.hi - sc};
      buf_store<1, true>(rAo, vo, 0u, a1);
      buf_store<1, true>(rHd, vo, 0u, h1);
      buf_store<1, true>(rHi, vo, 0u, i1);
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, px.de + det), dDe,
                                            t >= 1 ? (int)(sp * 4u) : kDeadOffset, 0, 0);
      sc = scn;
      st_p -= ch.pstep;
  };
  for (int s0 = 0; s0 < n; s0 += 2 * D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      // the loads of this ring slot were followed by at most D-1 steps' worth of memory operations
      wait_vmem<(D - 1) * kOps>();
      const auto px = ring[u];
      ring2[u] = load_next();
      __builtin_amdgcn_sched_barrier(0);  // the next pixel's loads go out before this step's work
      step(px, n - 1 - (s0 + u));
    }
    if (s0 + D >= n) break;  // wave-uniform
#pragma unroll
    for (int u = 0; u < D; ++u) {
      wait_vmem<(D - 1) * kOps>();
      const auto px = ring2[u];
      ring[u] = load_next();
      __builtin_amdgcn_sched_barrier(0);
      step(px, n - 1 - (s0 + D + u));
    }
  }
  }  // both walks of a fused pair
  if (p.dctx == nullptr) return;
  {
    const int F = (L + G - 1) / G;
    const bool valid = lane < G * L;
    const int g = valid ? lane / L : 0;
    const int cd = valid ? lane - g * L : 0;
#pragma unroll
    for (int i = 0; i < FM; ++i)
      if (valid && i < F && g * F + i < L) hist[(g * F + i) * L + cd] = hreg[i];
  }
  __syncthreads();
  // fold the pair table into dcontext's bins: |cd - fd| (1-D) or [min, max] (2-D), the diagonal
  // included (TRWP_backward_soft.cu:116-126)
  if (!p.ctx2d) {
    if (lane < L) {
      float acc = 0.f;
      for (int fd = 0; fd < L; ++fd) {
        if (fd + lane < L) acc += hist[fd * L + fd + lane];
        if (lane > 0 && fd - lane >= 0) acc += hist[fd * L + fd - lane];
      }
      if (acc != 0.f) atomicAdd(&p.dctx[lane], acc);
    }
  } else {
    for (int i = lane; i < LL; i += kWave) {
      const int fd = i / L, c2 = i - fd * L;
      if (c2 > fd) continue;  // handled by the (fd, cd) entry
      const float v = hist[i] + (c2 < fd ? hist[c2 * L + fd] : 0.f);
      if (v != 0.f) atomicAdd(&p.dctx[c2 * L + fd], v);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// More than 64 labels (up to 256, the label count the reference's stereo build accepts for
// ForwardSoft, TRWP_hard_soft/TRWP.cpp:336-340): R = ceil(L / 64) labels per lane, lane i owning
// labels i, i + 64, ...  A pixel's block of duals (L * L floats, up to 256 KB) does not fit in LDS,
// so it moves through a tile of kFc front labels at a time, tile[cd * kTs + fc], with an odd row
// stride: a lane reads and writes the row of its own label without bank conflicts, and the wave
// moves the tile to and from global memory in runs of kFc consecutive floats whatever the stored
// layout is (even directions [fd][cd], odd ones [cd][fd]).  1-D contexts only (2-D tables exist
// for at most 64 labels).  A step costs L * L exponentials, which dwarfs the latency of its loads:
// no prefetch ring here, the loads of a pixel are issued where they are needed.
// ------------------------------------------------------------------------------------------------
constexpr int kFc = 32;        // front labels per chunk of the tile
constexpr int kTs = kFc + 1;   // row stride of the tile (odd: conflict-free rows and columns)

// largest label among the lanes' labels (lane + 64 * j) whose predicate is set; dflt when none is
template <int R>
__device__ __forceinline__ int last_label_strided(const bool (&pred)[R], int dflt) {
  int best = dflt;
  bool found = false;
#pragma unroll
  for (int j = R - 1; j >= 0; --j) {
    const uint64_t m = ballot(pred[j]);
    if (!found && m != 0) {
      best = kWave * j + 63 - __builtin_clzll(m);
      found = true;
    }
  }
  return best;
}

// tile[cd * kTs + fc] <-> block entry (cd, fd = f0 + fc), nf = number of front labels in the chunk
template <int R>
__device__ __forceinline__ void tile_from_global(const float* __restrict__ blk, bool even, int L,
                                                 int f0, int nf, int lane, float* tile) {
  if (even) {  // stored [fd][cd]: consecutive lanes, consecutive labels
    for (int fc = 0; fc < nf; ++fc) {
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const int cd = lane + kWave * j;
        if (cd < L) tile[cd * kTs + fc] = __builtin_nontemporal_load(blk + (int64_t)(f0 + fc) * L + cd);
      }
    }
  } else {     // stored [cd][fd]: two rows of kFc front labels per wave access
    const int col = lane & (kFc - 1), sub = lane >> 5;
    for (int r0 = 0; r0 < L; r0 += 2) {
      const int row = r0 + sub;
      if (row < L && col < nf) tile[row * kTs + col] = __builtin_nontemporal_load(blk + (int64_t)row * L + f0 + col);
    }
  }
}

template <int R>
__device__ __forceinline__ void tile_to_global_rows(float* __restrict__ blk, int L, int f0, int nf,
                                                    int lane, const float* tile) {
  const int col = lane & (kFc - 1), sub = lane >> 5;
  for (int r0 = 0; r0 < L; r0 += 2) {
    const int row = r0 + sub;
    if (row < L && col < nf) __builtin_nontemporal_store(tile[row * kTs + col], blk + (int64_t)row * L + f0 + col);
  }
}

template <int R, bool TRAIN>
__global__ void __launch_bounds__(kWave) soft_wide_fwd_kernel(const SweepParams p) {
  extern __shared__ float smem[];
  const int L = p.L;
  float* a_s = smem;              // kMaxL
  float* ctx_s = a_s + kMaxL;     // kMaxL
  float* tile = ctx_s + kMaxL;    // L * kTs (training, odd directions)
  const int lane = threadIdx.x;
  const ChainCtx ch = locate_chain(p);
  if (ch.n < 2) return;  // nothing to write
  for (int i = lane; i < L; i += kWave) ctx_s[i] = p.ctx[i];
  __syncthreads();

  const int64_t HW = (int64_t)p.H * p.W;
  const int64_t P = (int64_t)p.B * HW;
  const int64_t N = P * L;
  const int dir = ch.dir;
  const bool even = (dir & 1) == 0;
  const int64_t img_p = (int64_t)ch.bv * HW;
  const float* __restrict__ bS = p.belief + img_p * L;
  const float* __restrict__ bMd = p.msg_in + (int64_t)dir * N + img_p * L;
  const float* __restrict__ bMi = p.msg_in + (int64_t)(dir ^ 1) * N + img_p * L;
  float* __restrict__ bMo = p.msg_out + (int64_t)dir * N + img_p * L;
  float* __restrict__ bSo = p.belief_out + img_p * L;
  const float* __restrict__ bW = p.edge + (int64_t)dir * P + img_p;
  float* __restrict__ bBlk = TRAIN ? p.edge_label + ((int64_t)dir * P + img_p) * L * L : nullptr;
  uint8_t* __restrict__ bInorm = TRAIN ? p.idx_norm + (int64_t)dir * P + img_p : nullptr;
  const float rho = p.rho;
  const float inf = INFINITY;

  int cd[R], cdc[R];
  bool valid[R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    cd[j] = lane + kWave * j;
    valid[j] = cd[j] < L;
    cdc[j] = valid[j] ? cd[j] : L - 1;  // keeps the table reads of idle lanes in range
  }

  float prev[R], uf[R];
  {
    const int64_t e0 = (int64_t)ch.pix0 * L;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      prev[j] = 0.f;
      uf[j] = inf;
      if (valid[j]) uf[j] = fmaf(bS[e0 + cd[j]] - bMd[e0 + cd[j]], rho, -bMi[e0 + cd[j]]);
    }
  }
  for (int t = 1; t < ch.n; ++t) {
    const int pix = ch.pix0 + t * ch.pstep;
    const int64_t e = (int64_t)pix * L;
    const float w = uniform_f(bW[pix]);
    float tt[R], un[R], a[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
      tt[j] = 0.f;
      un[j] = inf;
      if (valid[j]) {
        const float mi = bMi[e + cd[j]];
        tt[j] = bS[e + cd[j]] - bMd[e + cd[j]];
        un[j] = fmaf(tt[j], rho, -mi);  // UpdateUnaryKernelSoft, TRWP_forward_soft.cu:161-181
      }
      a[j] = fmaf(rho, prev[j], uf[j]);
      if (valid[j]) a_s[cd[j]] = a[j];
    }
    __syncthreads();
    // pass 1: minimum of the duals of each of the lane's labels (TRWP_forward_soft.cu:69-80)
    float mn[R], se[R], sd[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
      mn[j] = inf;
      se[j] = sd[j] = 0.f;
    }
#pragma unroll 2
    for (int fd = 0; fd < L; ++fd) {
      const float af = a_s[fd];
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const int k = cdc[j] - fd;
        mn[j] = fminf(mn[j], fmaf(w, ctx_s[k < 0 ? -k : k], af));
      }
    }
    // pass 2: softmin weights and the expected dual (:81-97); the block leaves chunk by chunk
    float* blk = TRAIN ? bBlk + (int64_t)pix * L * L : nullptr;
    for (int f0 = 0; f0 < L; f0 += kFc) {
      const int nf = L - f0 < kFc ? L - f0 : kFc;
      for (int fc = 0; fc < nf; ++fc) {
        const int fd = f0 + fc;
        const float af = a_s[fd];
#pragma unroll
        for (int j = 0; j < R; ++j) {
          const int k = cdc[j] - fd;
          const float dual = fmaf(w, ctx_s[k < 0 ? -k : k], af);
          const float ex = fast_exp(mn[j] - dual);
          se[j] += ex;
          sd[j] = fmaf(ex, dual, sd[j]);
          if (TRAIN && valid[j]) {
            if (even)
              __builtin_nontemporal_store(dual, blk + (int64_t)fd * L + cd[j]);  // [fd][cd]
            else
              tile[cd[j] * kTs + fc] = dual;
          }
        }
      }
      if (TRAIN && !even) {  // [cd][fd]: rows of the chunk, kFc consecutive floats each
        __syncthreads();
        tile_to_global_rows<R>(blk, L, f0, nf, lane, tile);
        __syncthreads();
      }
    }
    float soft[R], lo = inf;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      soft[j] = sd[j] / se[j];
      lo = fminf(lo, valid[j] ? soft[j] : inf);
    }
    const float nmin = wave_min(lo);
    bool pr[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const float m = soft[j] - nmin;
      pr[j] = valid[j] && (soft[j] == nmin);
      if (valid[j]) {
        __builtin_nontemporal_store(m, bMo + e + cd[j]);
        __builtin_nontemporal_store(tt[j] + m, bSo + e + cd[j]);
      }
      prev[j] = valid[j] ? m : 0.f;
      uf[j] = un[j];
    }
    if (TRAIN) {
      const int nidx = last_label_strided<R>(pr, L - 1);  // largest label on ties
      if (lane == 0) bInorm[pix] = (uint8_t)nidx;
    }
    __syncthreads();  // a_s is rewritten by the next step
  }
}

template <int R>
__global__ void __launch_bounds__(kWave) soft_wide_bwd_kernel(const BackParams p) {
  extern __shared__ float smem[];
  const int L = p.L;
  float* ctx_s = smem;           // kMaxL
  float* tile = ctx_s + kMaxL;   // L * kTs
  const int lane = threadIdx.x;
  const int64_t HW = (int64_t)p.H * p.W;
  const int64_t P = (int64_t)p.B * HW;
  const int64_t N = P * L;
  const ChainCtx ch = locate_chain(p);
  const int dir = ch.dir;
  const bool even = (dir & 1) == 0;
  const int n = ch.n;
  for (int i = lane; i < L; i += kWave) ctx_s[i] = p.ctx[i];
  __syncthreads();

  const int64_t img_p = (int64_t)ch.bv * HW;
  const bool read_h = !p.first_touch;
  const float* __restrict__ bA = p.a_in + img_p * L;
  float* __restrict__ bAo = p.a_out + img_p * L;
  float* __restrict__ bHd = p.h + (int64_t)dir * N + img_p * L;
  float* __restrict__ bHi = p.h + (int64_t)(dir ^ 1) * N + img_p * L;
  const float* __restrict__ bBlk = p.edge_label + ((int64_t)dir * P + img_p) * L * L;
  const uint8_t* __restrict__ bInorm = p.idx_norm + (int64_t)dir * P + img_p;
  const float* __restrict__ bW = p.edge + (int64_t)dir * P + img_p;
  float* __restrict__ bDe = p.dedge != nullptr ? p.dedge + (int64_t)dir * P + img_p : nullptr;
  const float rho = p.rho;
  const float inf = INFINITY;

  int cd[R], cdc[R];
  bool valid[R];
  float sc[R], hist[R];  // dU of the current pixel; dcontext bins lane + 64 * j
#pragma unroll
  for (int j = 0; j < R; ++j) {
    cd[j] = lane + kWave * j;
    valid[j] = cd[j] < L;
    cdc[j] = valid[j] ? cd[j] : L - 1;
    sc[j] = hist[j] = 0.f;
  }
  const int col = lane & (kFc - 1), sub = lane >> 5;

  for (int t = n - 1; t >= 0; --t) {
    const int pix = ch.pix0 + t * ch.pstep;
    const int64_t e = (int64_t)pix * L;
    float a[R], hd[R], hi[R], scn[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
      a[j] = hd[j] = hi[j] = scn[j] = 0.f;
      if (valid[j]) {
        a[j] = bA[e + cd[j]];
        if (read_h) {
          hd[j] = bHd[e + cd[j]];
          hi[j] = bHi[e + cd[j]];
        }
      }
    }
    float det = 0.f;
    if (t >= 1) {  // the chain start (t == 0) has no incoming edge
      const float w = uniform_f(bW[pix]);
      const int nidx = uniform_i((int)bInorm[pix]);
      float g[R], part = 0.f;
#pragma unroll
      for (int j = 0; j < R; ++j) {
        g[j] = valid[j] ? fmaf(rho, sc[j], a[j] + hd[j]) : 0.f;
        part += g[j];
      }
      const float tot = wave_sum(part);  // back norm, TRWP_backward_soft.cu:52-63
#pragma unroll
      for (int j = 0; j < R; ++j)
        if (cd[j] == nidx) g[j] -= tot;
      const float* blk = bBlk + (int64_t)pix * L * L;
      // pass A: softmin statistics of each of the lane's labels (:83-105), chunk by chunk with a
      // running minimum (the sums are rescaled when a chunk lowers it)
      float mn[R], se[R], sd[R];
#pragma unroll
      for (int j = 0; j < R; ++j) {
        mn[j] = inf;
        se[j] = sd[j] = 0.f;
      }
      for (int f0 = 0; f0 < L; f0 += kFc) {
        const int nf = L - f0 < kFc ? L - f0 : kFc;
        tile_from_global<R>(blk, even, L, f0, nf, lane, tile);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; ++j) {
          const float* row = tile + cdc[j] * kTs;
          float cm = inf;
          for (int fc = 0; fc < nf; ++fc) cm = fminf(cm, row[fc]);
          const float mnew = fminf(mn[j], cm);
          const float scale = fast_exp(mnew - mn[j]);  // 0 for the first chunk (mn = +inf)
          float s1 = se[j] * scale, s2 = sd[j] * scale;
          for (int fc = 0; fc < nf; ++fc) {
            const float x = row[fc];
            const float ex = fast_exp(mnew - x);
            s1 += ex;
            s2 = fmaf(ex, x, s2);
          }
          se[j] = s1;
          sd[j] = s2;
          mn[j] = mnew;
        }
        __syncthreads();
      }
      float gs[R], soft1[R], de = 0.f;
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const float inv = 1.f / se[j];
        soft1[j] = fmaf(sd[j], inv, 1.f);
        gs[j] = g[j] * inv;
      }
      // pass B: ddual = g * prob * (1 - dual + soft) (:110-113) replaces the duals in the tile;
      // its column sums are dU[q, fd], its diagonal sums the dcontext bins
#pragma unroll
      for (int jc = 0; jc < R; ++jc) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int f0 = kWave * jc + kFc * half;
          if (f0 < L) {  // wave-uniform
            const int nf = L - f0 < kFc ? L - f0 : kFc;
            tile_from_global<R>(blk, even, L, f0, nf, lane, tile);
            __syncthreads();
#pragma unroll
            for (int j = 0; j < R; ++j) {
              if (valid[j]) {
                float* row = tile + cd[j] * kTs;
                for (int fc = 0; fc < nf; ++fc) {
                  const float x = row[fc];
                  const float dd = gs[j] * fast_exp(mn[j] - x) * (soft1[j] - x);
                  const int k = cd[j] - (f0 + fc);
                  de = fmaf(ctx_s[k < 0 ? -k : k], dd, de);
                  row[fc] = dd;
                }
              }
            }
            __syncthreads();
            // dU[q, f0 + col]: every lane adds up half of the rows of its column
            float cs = 0.f;
            if (col < nf)
              for (int r = sub; r < L; r += 2) cs += tile[r * kTs + col];
            cs += __shfl_xor(cs, 32);
            if (sub == half) scn[jc] += cs;  // label f0 + col = lane + 64 * jc
            // dcontext[k] += w * ddual over |cd - fd| == k (the pairs with k == 0 included,
            // TRWP_backward_soft.cu:116-126): lane + 64 * j owns bin k
            if (p.dctx != nullptr) {
#pragma unroll
              for (int j = 0; j < R; ++j) {
                const int k = cd[j];
                if (k < L) {
                  float acc = 0.f;
                  for (int fc = 0; fc < nf; ++fc) {
                    const int fd = f0 + fc;
                    if (fd + k < L) acc += tile[(fd + k) * kTs + fc];
                    if (k > 0 && fd - k >= 0) acc += tile[(fd - k) * kTs + fc];
                  }
                  hist[j] = fmaf(w, acc, hist[j]);
                }
              }
            }
            __syncthreads();
          }
        }
      }
      det = wave_sum(de);
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
      if (valid[j]) {
        const float an = fmaf(rho, sc[j], a[j]);  // g_k += rho*dU for every k, dunary too
        bAo[e + cd[j]] = an;
        bHd[e + cd[j]] = -an;             // g_dir = 0 after its sweep
        bHi[e + cd[j]] = hi[j] - sc[j];   // g_inv -= dU
      }
      sc[j] = scn[j];
    }
    if (t >= 1 && bDe != nullptr && lane == 0) bDe[pix] += det;
  }
  if (p.dctx != nullptr) {
#pragma unroll
    for (int j = 0; j < R; ++j)
      if (valid[j] && hist[j] != 0.f) atomicAdd(&p.dctx[cd[j]], hist[j]);
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

// dwords per lane that cover a pixel's block of duals in the one-label-per-lane kernels (33 to 64
// labels: up to 64)
int tile_bucket(int) { return kWave; }

}  // namespace

void launch_soft_fwd(const SweepParams& p, bool train, hipStream_t st) {
  const int blocks = p.block_prefix[p.n_dirs];
  if (blocks <= 0) return;
  if (p.L > kWave) {  // several labels per lane
    const size_t wide_lds = sizeof(float) * (2 * kMaxL + (train ? p.L * kTs : 0));
    const int R = (p.L + kWave - 1) / kWave;
#define MPL_SOFT_WIDE_FWD(RR)                                                       \
  do {                                                                              \
    if (train)                                                                      \
      soft_wide_fwd_kernel<RR, true><<<blocks, kWave, wide_lds, st>>>(p);           \
    else                                                                            \
      soft_wide_fwd_kernel<RR, false><<<blocks, kWave, wide_lds, st>>>(p);          \
  } while (0)
    if (R == 2)
      MPL_SOFT_WIDE_FWD(2);
    else if (R == 3)
      MPL_SOFT_WIDE_FWD(3);
    else
      MPL_SOFT_WIDE_FWD(4);
#undef MPL_SOFT_WIDE_FWD
    return;
  }
  const int LL = p.L * p.L;
  const int T = tile_bucket(p.L);
  const size_t lds = sizeof(float) * (LL + (train ? (LL > kWave * T ? LL : kWave * T) : 0));
  if (p.L <= 32) {  // front labels split over the idle lanes
#define MPL_SOFT_SPLIT_FWD(GG, FF, NN)                                                       \
  do {                                                                                       \
    const size_t slds = sizeof(float) * (LL + (train ? 256 * NN + kWave : 0));               \
    if (train)                                                                               \
      soft_split_fwd_kernel<true, GG, FF, NN><<<blocks, kWave, slds, st>>>(p);               \
    else                                                                                     \
      soft_split_fwd_kernel<false, GG, FF, NN><<<blocks, kWave, slds, st>>>(p);              \
  } while (0)
    if (p.L <= 16)
      MPL_SOFT_SPLIT_FWD(4, 4, 1);
    else if (p.L <= 21)
      MPL_SOFT_SPLIT_FWD(3, 7, 2);
    else
      MPL_SOFT_SPLIT_FWD(2, 16, 4);
#undef MPL_SOFT_SPLIT_FWD
    return;
  }
  if (!train)
    soft_fwd_kernel<false, 0><<<blocks, kWave, lds, st>>>(p);
  else
    soft_fwd_kernel<true, kWave><<<blocks, kWave, lds, st>>>(p);
}

void launch_soft_bwd(const BackParams& p, hipStream_t st) {
  const int blocks = p.block_prefix[p.n_dirs];
  if (blocks <= 0) return;
  if (p.L > kWave) {  // several labels per lane
    const size_t wide_lds = sizeof(float) * (kMaxL + p.L * kTs);
    const int R = (p.L + kWave - 1) / kWave;
    if (R == 2)
      soft_wide_bwd_kernel<2><<<blocks, kWave, wide_lds, st>>>(p);
    else if (R == 3)
      soft_wide_bwd_kernel<3><<<blocks, kWave, wide_lds, st>>>(p);
    else
      soft_wide_bwd_kernel<4><<<blocks, kWave, wide_lds, st>>>(p);
    return;
  }
  const int LL = p.L * p.L;
  const int T = tile_bucket(p.L);
  const size_t lds = sizeof(float) * (2 * LL + kWave * T + p.L * (p.L | 1));
  if (p.L <= 32) {  // front labels split over the idle lanes
    const int NQ = p.L <= 16 ? 4 : (p.L <= 21 ? 6 : 8);
    const size_t slds = sizeof(float) * (2 * ((LL + 3) & ~3) + p.L * 4 * NQ + kWave);
    if (p.L <= 16)
      soft_split_bwd_kernel<4, 4, 4><<<blocks, kWave, slds, st>>>(p);
    else if (p.L <= 21)
      soft_split_bwd_kernel<3, 7, 6><<<blocks, kWave, slds, st>>>(p);
    else
      soft_split_bwd_kernel<2, 16, 8><<<blocks, kWave, slds, st>>>(p);
    return;
  }
  // up to 66 KB of LDS at 64 labels: above the default limit of a workgroup
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&soft_bwd_kernel<kWave>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  soft_bwd_kernel<kWave><<<blocks, kWave, lds, st>>>(p);
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
