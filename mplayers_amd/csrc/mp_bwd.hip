// Reverse scan of TRWP / ISGMR for gfx950: one wavefront per chain, see mp_common.h.
//
// Follows HorizontalKernelBack / DiagonalKernelWideBack / DiagonalKernelNarrowBack
// (TRWP_backward.cu:49-275, ISGMR_backward.cu:62-288) fused with UpdateUnaryKernelBack
// (TRWP_backward.cu:26-47) and the memsets after it (:421-422).  Per pixel p, visited in reverse
// chain order, with g the gradient w.r.t. the normalised message of p:
//     g[norm_index[p]] -= sum(g)                                    (MsgNormNaiveBack)
//     for cd: fd = min_index[p, cd];  dU[q, fd] += g[cd];  g_dir[q, fd] += rho * g[cd]
//             dedge[p] += ctx(cd, fd) * g[cd];  dctx[ctx index] += w[p] * g[cd]  if cd != fd
// The scatter target dU[q, :] stays in LDS/registers: it is the only thing the next step needs.
//
// TRWP keeps the per-direction gradient planes as g_k = A + h_k (A ends up being dunary), so the
// "for all k" updates of UpdateUnaryKernelBack touch one plane instead of n_dir.
//
// Compiled once per R (labels per lane) with -DMPL_INST_R=<R>.

#include "mp_common.h"

namespace mpl {
namespace {

// Several labels per lane, and 33 to 64 labels in launches that fill the chip: an LDS float atomic
// and the exchange that reads its sums back take some 250 clocks and occupy the LDS of the CU, so
// the common cases of the scatter and of the dcontext histogram are done without them:
//   * argmin indices that point at the two most popular targets of the pixel (taken from the first
//     and the last label; with a truncated pairwise term nearly every label points at argmin(a))
//     are summed with a wave reduction,
//   * indices within kNear labels of their own label are moved with DPP label shifts,
//   * only what is left goes through LDS atomics.
// One label per lane otherwise (DIRECT): the step is bound by its own latency, and one atomic for
// the scatter, one exchange and one atomic for the histogram are the shortest way through it.
constexpr int kNear = 3;
// (launches of at most LaunchPolicy::direct_max_chains chains are taken to be latency-bound)

template <int R>
struct PixB {
  float a[R], hd[R], hi[R];
  int fd[R];
  int nidx;
  float w, de;
};

// DIRECT: one label per lane, everything through the LDS accumulators (see above and the launcher)
// GRAD: bit 0 = dedge_weights is wanted, bit 1 = dcontext is wanted (a caller with a fixed pairwise
// table or edge weights that are not learned passes null for them; that part of the step is then
// not compiled in: no dedge read-modify-write, no context products, no histogram gathers)
template <int R, bool VEC, bool MASK, bool JACOBI, bool DIRECT, int GRAD>
__global__ void __launch_bounds__(kWave) sweep_bwd_kernel(const BackParams p) {
  constexpr bool DE = (GRAD & 1) != 0, DC = (GRAD & 2) != 0;
  extern __shared__ float smem[];
  const int L = p.L;
  // 2-D context tables exist for at most 64 labels, i.e. only with one label per lane
  const bool ctx2d = (R == 1) && p.ctx2d;
  const int n_ctx = ctx2d ? L * L : L;
  float* sc_s = smem;              // kMaxL floats: scatter target of the slow path
  // weighted gradients of popular class 0 by label, with L zeros on either side so that the
  // gather at label f +- k needs no range checks: 3 * L floats, data at [L, 2L)
  float* g0_s = sc_s + kMaxL;
  float* g1_s = g0_s + 3 * L;      // same for class 1
  float* ctx_s = g1_s + 3 * L;     // context table
  float* hist_s = ctx_s + n_ctx;   // dcontext accumulator of the slow path (and of 2-D contexts)
  const int lane = threadIdx.x;
  const int64_t P = (int64_t)p.B * p.H * p.W;
  const int64_t N = P * L;
  const ChainCtx ch0 = locate_chain(p);
  const int n = ch0.n;

  const bool same = DC && p.same_label != 0;
  for (int i = lane; i < n_ctx; i += kWave) {
    ctx_s[i] = p.ctx[i];
    hist_s[i] = 0.f;
  }
  for (int i = lane; i < kMaxL + 6 * L; i += kWave) sc_s[i] = 0.f;  // sc_s, g0_s, g1_s
  __syncthreads();

  // Offsets |fd - cd| come from the band of the context (entries below its constant tail) or from
  // the far candidate, which is nearly always one of the popular targets.  A 1-D context with a
  // band of K entries therefore needs label shifts up to K - 1 only; rarer offsets within kNear
  // fall through to the slow path, so any choice here is exact.
  // (With one label per lane the step is short and the scans are bound by its latency, which
  // the wave-uniform branches would lengthen: the narrowing is for several labels per lane.)
  int near_max = kNear;
  if (R > 1 && !ctx2d) {
    int kb = 0;
    for (int i = lane; i < L; i += kWave) kb = (ctx_s[i] != ctx_s[L - 1]) ? i + 1 : kb;
    kb = (int)-wave_min(-(float)kb);  // wave maximum: entries at and beyond kb equal the last one
    near_max = kb - 1 < 1 ? 1 : (kb - 1 > kNear ? kNear : kb - 1);
  }

  const int lab0 = R * lane;
  bool valid[R];
#pragma unroll
  for (int j = 0; j < R; ++j) valid[j] = MASK ? (lab0 + j < L) : true;
  float hist_reg[R];        // dcontext[label] partial sums of this lane's own labels (1-D context)
  float near_acc[kNear + 1];  // dcontext[k] partial sums for k <= kNear (1-D context)
#pragma unroll
  for (int j = 0; j < R; ++j) hist_reg[j] = 0.f;
#pragma unroll
  for (int k = 0; k <= kNear; ++k) near_acc[k] = 0.f;

  // Gauss-Seidel, chain-starved launches (p.fused_pair): the wavefront walks its chain for the odd
  // direction and then, over the same pixels in reverse, for the even one, which the next launch
  // would otherwise do; what the first walk stored is read back by the same wavefront in program
  // order, and dcontext is collected over both walks and flushed once.
  const int halves = (!JACOBI && p.fused_pair) ? 2 : 1;
#pragma clang loop unroll(disable)
  for (int half = 0; half < halves; ++half) {
  ChainCtx ch = ch0;
  bool first_touch = p.first_touch != 0, inv_a = p.inv_from_a != 0;
  bool skip_hd_store = p.skip_hd_store != 0, skip_hi_store = p.skip_hi_store != 0;
  const float* a_in = p.a_in;
  if (half) {
    ch.dir = ch0.dir ^ 1;
    ch.pix0 = ch0.pix0 + (n - 1) * ch0.pstep;
    ch.pstep = -ch0.pstep;
    first_touch = false;
    inv_a = true;  // the walk before this one swept the opposite direction
    skip_hd_store = skip_hi_store = p.skip_h2 != 0;
    a_in = p.a_out;
    wait_vmem<0>();
    __syncthreads();
  }
  const int dir = ch.dir;
  const int64_t HW = (int64_t)p.H * p.W;
  const int64_t img_p = (int64_t)ch.bv * HW;  // first pixel of this batch item
  const int64_t img_e = img_p * L;
  const int vbytes = L * 4;
  const bool read_h = !JACOBI && !first_touch;
  const bool inv_from_a = !JACOBI && inv_a;
  // plane bases of this batch item and direction; label-vector descriptors are formed per access
  const float* __restrict__ bA =
      (JACOBI ? p.gu_in + (int64_t)(p.gu_pair_share ? (dir & ~1) : dir) * p.gu_stride : a_in) +
      img_e;
  float* __restrict__ bAo = (JACOBI ? p.du_out + (int64_t)dir * N : p.a_out) + img_e;
  float* hbase = JACOBI ? p.du_out : p.h;  // Jacobi never touches these two planes
  float* __restrict__ bHd = hbase + (int64_t)dir * N + img_e;
  float* __restrict__ bHi = hbase + (int64_t)(dir ^ 1) * N + img_e;
  const uint8_t* __restrict__ bImin = p.idx_min + (int64_t)dir * N + img_e;
  const int img_bytes_p = (int)(HW * 4 > 0x7fffffff ? 0x7fffffff : HW * 4);
  const rsrc_t dInorm = make_rsrc(p.idx_norm + (int64_t)dir * P + img_p, (int)HW);
  const rsrc_t dW = make_rsrc(p.edge + (int64_t)dir * P + img_p, img_bytes_p);
  const rsrc_t dDe = make_rsrc(DE ? p.dedge + (int64_t)dir * P + img_p : nullptr, DE ? img_bytes_p : 0);
  const float rho = p.rho;
  const int foff = lab0 * 4;

  // VEC: one descriptor per plane for the whole kernel, covering the batch item's image; a lane
  // reaches its labels of a pixel through its vector offset, a lane without labels (or a step that
  // must not store) through an offset no descriptor covers: one multiply, one add and one select
  // per pixel instead of a descriptor formed per access.  Planes that are not to be read or stored
  // get an empty descriptor.
  const bool lane_ok = !MASK || lab0 < L;
  const int img_bytes = (int)(unsigned)(HW * L * 4);
  const rsrc_t rA = make_rsrc(bA, img_bytes);
  const rsrc_t rAo = make_rsrc(bAo, img_bytes);
  const rsrc_t rHdIn = make_rsrc(bHd, (!JACOBI && read_h) ? img_bytes : 0);
  const rsrc_t rHiIn = make_rsrc(bHi, (!JACOBI && read_h && !inv_from_a) ? img_bytes : 0);
  const rsrc_t rHdOut = make_rsrc(bHd, (JACOBI || skip_hd_store) ? 0 : img_bytes);
  const rsrc_t rHiOut = make_rsrc(bHi, (JACOBI || skip_hi_store) ? 0 : img_bytes);
  const rsrc_t rImin = make_rsrc(bImin, (int)(HW * L));
  // loads run from the last pixel of the chain down to the first; past it the first is refetched
  // (VEC: the prefetch simply runs on; what lies there is another pixel or reads as 0)
  int ld_t = n - 1;
  int ld_p = ch.pix0 + (n - 1) * ch.pstep;
  auto load_next = [&]() __attribute__((always_inline)) {
    PixB<R> r;
    const unsigned pp = (unsigned)uniform_i((VEC || ld_t >= 0) ? ld_p : ch.pix0);
    const unsigned so = pp * (unsigned)vbytes;
    if constexpr (VEC) {
      const int vo = (int)(lane_ok ? so + (unsigned)foff : kDeadWide);
      buf_load<R, true>(rA, vo, 0u, r.a);
      if (!JACOBI) {
        // before the first write of these planes they count as zero (empty descriptor); the sweep
        // that ran just before this one was the opposite direction's and left h_inv = -A
        buf_load<R, true>(rHdIn, vo, 0u, r.hd);
        buf_load<R, true>(rHiIn, vo, 0u, r.hi);
      }
      buf_load_u8<R, true>(rImin, (int)(lane_ok ? pp * (unsigned)L + (unsigned)lab0 : kDeadWide), 0u,
                           r.fd);
    } else {
      const int nrec = (int)(so + (unsigned)vbytes);
      buf_load<R, VEC>(make_rsrc(bA, nrec), foff, so, r.a);
      if (!JACOBI) {
        // before the first write of these planes they count as zero: an empty descriptor reads 0
        buf_load<R, VEC>(make_rsrc(bHd, read_h ? nrec : 0), foff, so, r.hd);
        // the sweep that ran just before this one was the opposite direction's: it left
        // h_inv = -A everywhere, so the plane need not be read (empty descriptor, no traffic)
        buf_load<R, VEC>(make_rsrc(bHi, (read_h && !inv_from_a) ? nrec : 0), foff, so, r.hi);
      }
      buf_load_u8<R, VEC>(make_rsrc(bImin, (int)(pp * (unsigned)L + (unsigned)L)), lab0,
                          pp * (unsigned)L, r.fd);
    }
    // (no arithmetic on what was just loaded in here: it would have to wait for the loads, and the
    // compiler places such work at the end of the loop body, where the wait drains the whole queue)
    if (JACOBI) {
#pragma unroll
      for (int j = 0; j < R; ++j) r.hd[j] = r.hi[j] = 0.f;
    }
    r.nidx = __builtin_amdgcn_raw_buffer_load_b8(dInorm, (int)pp, 0, 0);
    r.w = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dW, (int)(pp * 4u), 0, 0));
    r.de = 0.f;
    if (DE)
      r.de = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dDe, (int)(pp * 4u), 0, 0));
    ld_t -= 1;
    ld_p -= ch.pstep;
    return r;
  };

  // memory instructions per step: label vectors, indices, norm index, weight, dedge in;
  // label vectors and dedge out
  constexpr int kOps = (JACOBI ? 1 : 3) * vec_ops(R, VEC) + byte_ops(R, VEC) + 2 + (DE ? 1 : 0) +
                       (JACOBI ? 1 : 3) * vec_ops(R, VEC) + (DE ? 1 : 0);
  constexpr int D = ring_depth(kOps);
  // two banks of D pixels in flight, consumed in turn: after 2 D steps every value sits in the
  // register it started in (a single bank ends the loop in one register move per value in flight)
  PixB<R> ring[D], ring2[D];
#pragma unroll
  for (int u = 0; u < D; ++u) {
    ring[u] = load_next();
    // keeps the pixels' loads in this order: the compiler's own waits in the loop are sized for
    // the order it sees here, and a later pixel's loads placed first would make them drain the queue
    MPL_ORDER_LOADS();
  }

  float sc[R];  // dU of the current pixel: what the previous step scattered into it
#pragma unroll
  for (int j = 0; j < R; ++j) sc[j] = 0.f;
  const int last_lane = (L - 1) / R, last_reg = (L - 1) % R;

  int st_p = ch.pix0 + (n - 1) * ch.pstep;
  auto step = [&](const PixB<R>& px, const int t) __attribute__((always_inline)) {
      float scn[R];
#pragma unroll
      for (int j = 0; j < R; ++j) scn[j] = 0.f;
      float det = 0.f;
      if (t >= 1) {  // the chain start (t == 0) has no incoming edge
        const float w = uniform_f(px.w);
        const int nidx = __builtin_amdgcn_readfirstlane(px.nidx);
        float gv[R];
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
          // gradient w.r.t. the normalised message of this pixel, including what the previous
          // step added through the recurrence (dmsg[front] += rho * value, TRWP_backward.cu:108)
          float base = JACOBI ? px.a[j] : (px.a[j] + px.hd[j]);
          gv[j] = valid[j] ? fmaf(rho, sc[j], base) : 0.f;
          part += gv[j];
        }
        // MsgNormNaiveBack, commonCUDA.cuh:131-145
        const float tot = R == 1 ? wave_sum_fast(part) : wave_sum(part);
        if constexpr (R == 1 && DIRECT) {
          // one atomic that scatters the gradients to their argmin labels, one exchange that
          // reads the sums back and clears them, one atomic for the dcontext histogram
          const int cd = lane, fd = px.fd[0];
          const int ao = fd > cd ? fd - cd : cd - fd;
          const int ci = !valid[0] ? 0 : (ctx2d ? (int)__umul24(min(cd, fd), L) + max(cd, fd) : ao);
          const float cv = DE ? ctx_s[ci] : 0.f;
          float g = gv[0];
          if (cd == nidx) g -= tot;
          float dev = valid[0] ? cv * g : 0.f;
          asm volatile("" : "+v"(dev));  // (formed here, not behind the atomics)
          // The table entry is there before the atomics are issued, so the sum of dedge below runs
          // while they are under way.  The LDS executes the instructions of a wavefront in their
          // order: the exchange finds the sums complete without a wait in between, and the
          // histogram's atomic, which nothing waits for, queues up behind it.  The three are
          // relaxed atomics to different addresses per lane, which the compiler may reorder: the
          // fences at wavefront scope forbid that and emit no instruction.
          __builtin_amdgcn_wave_barrier();
          if (valid[0]) {
            atomicAdd(&sc_s[fd], g);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            scn[0] = atomicExch(&sc_s[lane], 0.f);  // read and clear
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            if (DC && (same || cd != fd)) atomicAdd(&hist_s[ci], w * g);
          }
          if (DE) det = wave_sum_fast(dev);
        } else {
        // the two popular targets: where the first and the last label point
        const int f0 = __builtin_amdgcn_readlane(px.fd[0], 0);
        int f1 = 0;
#pragma unroll
        for (int j = 0; j < R; ++j) {
          int v = __builtin_amdgcn_readlane(px.fd[j], last_lane);
          f1 = (j == last_reg) ? v : f1;
        }
        // off[j] = front label - own label; kPopular marks labels whose front label is one of the
        // two popular targets (they are summed with wave reductions instead of being moved)
        constexpr int kPopular = 0x4000;
        int off[R];
        float p0 = 0.f, p1 = 0.f, de = 0.f;
        bool any_left = false;
#pragma unroll
        for (int j = 0; j < R; ++j) {
          const int cd = lab0 + j, fd = px.fd[j];
          if (cd == nidx) gv[j] -= tot;
          const int d = fd - cd;
          const int ao = d < 0 ? -d : d;
          const bool c0 = fd == f0;
          const bool c1 = (fd == f1) & !c0;
          p0 += c0 ? gv[j] : 0.f;
          p1 += c1 ? gv[j] : 0.f;
          off[j] = (c0 | c1) ? kPopular : d;
          any_left |= !(c0 | c1) & (ao > near_max) & valid[j];
          // dedge_weights[cur] += ctx(cd, fd) * value
          if (DE) {
            const int ci = !valid[j] ? 0 : (ctx2d ? (cd < fd ? cd * L + fd : fd * L + cd) : ao);
            de = fmaf(ctx_s[ci], gv[j], de);
          }
        }
        const float s0sum = wave_sum(p0);
        // nothing belongs to the second class when both popular targets coincide (the usual case)
        float s1sum = 0.f;
        if (R == 1 || f1 != f0) s1sum = wave_sum(p1);
        // near targets: sc_next[l] += g[l - o] where index(l - o) == l, |o| <= kNear
        float tp[R], tn[R], near_t[kNear + 1];
#pragma unroll
        for (int j = 0; j < R; ++j) tp[j] = tn[j] = 0.f;
#pragma unroll
        for (int o = kNear; o >= 1; --o) {
          near_t[o] = 0.f;
          if (R > 1 && o > near_max) continue;  // wave-uniform
#pragma unroll
          for (int j = 0; j < R; ++j) {
            const float cp = (off[j] == o) ? gv[j] : 0.f;
            const float cn = (off[j] == -o) ? gv[j] : 0.f;
            near_t[o] += cp + cn;
            tp[j] += cp;
            tn[j] += cn;
          }
          // move one label up (tp) / down (tn)
          const float up_in = wave_shr1(tp[R - 1], 0.f);
          const float dn_in = wave_shl1(tn[0], 0.f);
#pragma unroll
          for (int j = R - 1; j > 0; --j) tp[j] = tp[j - 1];
          tp[0] = up_in;
#pragma unroll
          for (int j = 0; j < R - 1; ++j) tn[j] = tn[j + 1];
          tn[R - 1] = dn_in;
        }
#pragma unroll
        for (int j = 0; j < R; ++j) {
          const int cd = lab0 + j;
          const float own = (off[j] == 0) ? gv[j] : 0.f;
          scn[j] = own + tp[j] + tn[j] + (cd == f0 ? s0sum : 0.f) + (cd == f1 ? s1sum : 0.f);
        }
        // dcontext += edge_weight * value where cd != fd (TRWP_backward.cu:111-112); with `same`
        // also where cd == fd (TRWP_hard_soft/TRWP_backward.cu:110)
        if (!DC) {
        } else if (!ctx2d) {
          // bin 0, labels outside the popular classes that point at themselves
          if (same) {  // wave-uniform
            float own_sum = 0.f;
#pragma unroll
            for (int j = 0; j < R; ++j) own_sum += (off[j] == 0) ? gv[j] : 0.f;
            near_acc[0] = fmaf(w, own_sum, near_acc[0]);
          }
#pragma unroll
          for (int o = 1; o <= kNear; ++o) near_acc[o] = fmaf(w, near_t[o], near_acc[o]);
          // popular classes: bin |cd - f| is reached from labels f + k and f - k; gather through LDS
          // (bin 0 collects the popular label's own value twice: halved when it is flushed)
#pragma unroll
          for (int j = 0; j < R; ++j)
            if (valid[j]) g0_s[L + lab0 + j] = (px.fd[j] == f0) ? w * gv[j] : 0.f;
          __syncthreads();
#pragma unroll
          for (int j = 0; j < R; ++j) {
            const int k = valid[j] ? lab0 + j : 0;
            hist_reg[j] += g0_s[L + f0 + k] + g0_s[L + f0 - k];
          }
          if (f1 != f0) {
#pragma unroll
            for (int j = 0; j < R; ++j)
              if (valid[j]) g1_s[L + lab0 + j] = (px.fd[j] == f1) ? w * gv[j] : 0.f;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < R; ++j) {
              const int k = valid[j] ? lab0 + j : 0;
              hist_reg[j] += g1_s[L + f1 + k] + g1_s[L + f1 - k];
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < R; ++j) {
            const int cd = lab0 + j, fd = px.fd[j];
            if (valid[j] && (same || cd != fd))
              atomicAdd(&hist_s[cd < fd ? cd * L + fd : fd * L + cd], w * gv[j]);
          }
        }
        // whatever is neither popular nor near: LDS atomics
        if (ballot(any_left) != 0) {
#pragma unroll
          for (int j = 0; j < R; ++j) {
            const int ao = off[j] < 0 ? -off[j] : off[j];
            if (valid[j] && off[j] != kPopular && ao > near_max) {
              atomicAdd(&sc_s[px.fd[j]], gv[j]);
              if (DC && !ctx2d) atomicAdd(&hist_s[ao], w * gv[j]);
            }
          }
          __syncthreads();
#pragma unroll
          for (int j = 0; j < R; ++j)
            if (valid[j]) scn[j] += atomicExch(&sc_s[lab0 + j], 0.f);  // read and clear
        }
        if (DE) det = wave_sum(de);
        }
      }
      // pixel-local part of UpdateUnaryKernelBack with dU[pix] = sc; nothing is stored for t < 0
      const unsigned sp = (unsigned)uniform_i(st_p);
      const unsigned so = sp * (unsigned)vbytes;
      const int nrec = t >= 0 ? (int)(so + (unsigned)vbytes) : 0;
      const int vo = (int)((lane_ok && t >= 0) ? so + (unsigned)foff : kDeadWide);
      if (JACOBI) {
        if constexpr (VEC)
          buf_store<R, true>(rAo, vo, 0u, sc);
        else
          buf_store<R, VEC>(make_rsrc(bAo, nrec), foff, so, sc);
      } else {
        float an[R], hdn[R], hin[R];
#pragma unroll
        for (int j = 0; j < R; ++j) {
          an[j] = fmaf(rho, sc[j], px.a[j]);  // g_k += rho*dU for every k, dunary too
          hdn[j] = -an[j];                    // g_dir = 0 after its sweep
          // g_inv -= dU; after the opposite direction's sweep g_inv is -A and was not read
          hin[j] = (inv_from_a ? -px.a[j] : px.hi[j]) - sc[j];
        }
        // h_dir = -A is only read by the next launch when that one sweeps the opposite
        // direction, which derives it from A instead: nothing is stored then (nor after the last
        // sweeps of the pass, whose h planes nobody reads)
        if constexpr (VEC) {
          buf_store<R, true>(rAo, vo, 0u, an);
          buf_store<R, true>(rHdOut, vo, 0u, hdn);
          buf_store<R, true>(rHiOut, vo, 0u, hin);
        } else {
          buf_store<R, VEC>(make_rsrc(bAo, nrec), foff, so, an);
          buf_store<R, VEC>(make_rsrc(bHd, skip_hd_store ? 0 : nrec), foff, so, hdn);
          buf_store<R, VEC>(make_rsrc(bHi, skip_hi_store ? 0 : nrec), foff, so, hin);
        }
      }
      // each pixel receives over exactly one edge per direction: plain read-modify-write
      if (DE)
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, px.de + det), dDe,
                                              t >= 1 ? (int)(sp * 4u) : kDeadOffset, 0, 0);
#pragma unroll
      for (int j = 0; j < R; ++j) sc[j] = scn[j];
      st_p -= ch.pstep;
  };
  for (int s0 = 0; s0 < n; s0 += 2 * D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      // the loads of this ring slot were followed by at most D-1 steps' worth of memory operations
      wait_vmem<(D - 1) * kOps>();
      const PixB<R> px = ring[u];
      ring2[u] = load_next();
      step(px, n - 1 - (s0 + u));
    }
    if (s0 + D >= n) break;  // wave-uniform
#pragma unroll
    for (int u = 0; u < D; ++u) {
      wait_vmem<(D - 1) * kOps>();
      const PixB<R> px = ring2[u];
      ring[u] = load_next();
      step(px, n - 1 - (s0 + D + u));
    }
  }
  }  // both walks of a fused pair
  if (!DC) return;
  __syncthreads();
  for (int i = lane; i < n_ctx; i += kWave) {
    float v = hist_s[i];
    if (v != 0.f) atomicAdd(&p.dctx[i], v);
  }
  if (!ctx2d) {
#pragma unroll
    for (int j = 0; j < R; ++j)
      if (valid[j] && lab0 + j >= 1 && hist_reg[j] != 0.f) atomicAdd(&p.dctx[lab0 + j], hist_reg[j]);
#pragma unroll
    for (int k = 1; k <= kNear; ++k) {
      const float v = wave_sum(near_acc[k]);
      if (lane == 0 && k < L && v != 0.f) atomicAdd(&p.dctx[k], v);
    }
    if (same) {
      // bin 0: the popular labels that point at themselves were gathered twice into the
      // accumulator of label 0 (x + x, exact), the others were summed per lane
      const float v = wave_sum(near_acc[0] + (lane == 0 ? 0.5f * hist_reg[0] : 0.f));
      if (lane == 0 && v != 0.f) atomicAdd(&p.dctx[0], v);
    }
  }
}

template <int R, bool VEC, bool MASK, int GRAD>
void launch_vmg(const BackParams& p, bool jacobi, hipStream_t st) {
  const int blocks = p.block_prefix[p.n_dirs];
  const size_t lds = sizeof(float) * (kMaxL + 6 * p.L + 2 * (p.ctx2d ? p.L * p.L : p.L));
  if constexpr (R == 1) {
    // Through the accumulators: up to 32 labels (with few lanes of a wavefront in use the atomics
    // are short even where several wavefronts share a SIMD: 8 x 400 x 400, min(k, 3) table, TRWP
    // fwd+bwd with 16 / 24 / 32 labels 5.7 / 8.2 / 7.7 ms against 9.2 / 10.6 / 9.5 with the
    // shortcuts), 2-D tables (their argmin labels are spread over all labels), and 33 to 64 labels
    // while the launch is latency-bound (40 labels, 1200 chains per launch 3.4 against 4.7 ms, but
    // 64 labels, 3200 chains 9.0 against 7.5).
    if (p.L <= kPackedMaxL || p.ctx2d || blocks <= launch_policy().direct_max_chains) {
      if (jacobi)
        sweep_bwd_kernel<R, VEC, MASK, true, true, GRAD><<<blocks, kWave, lds, st>>>(p);
      else
        sweep_bwd_kernel<R, VEC, MASK, false, true, GRAD><<<blocks, kWave, lds, st>>>(p);
      return;
    }
  }
  if (jacobi)
    sweep_bwd_kernel<R, VEC, MASK, true, false, GRAD><<<blocks, kWave, lds, st>>>(p);
  else
    sweep_bwd_kernel<R, VEC, MASK, false, false, GRAD><<<blocks, kWave, lds, st>>>(p);
}

template <int R, bool VEC, bool MASK>
void launch_vm(const BackParams& p, bool jacobi, hipStream_t st) {
  switch ((p.dedge != nullptr ? 1 : 0) | (p.dctx != nullptr ? 2 : 0)) {
    case 0: launch_vmg<R, VEC, MASK, 0>(p, jacobi, st); break;
    case 1: launch_vmg<R, VEC, MASK, 1>(p, jacobi, st); break;
    case 2: launch_vmg<R, VEC, MASK, 2>(p, jacobi, st); break;
    default: launch_vmg<R, VEC, MASK, 3>(p, jacobi, st); break;
  }
}

}  // namespace

template <int R>
void launch_sweep_bwd(const BackParams& p, bool jacobi, hipStream_t st) {
  if (p.block_prefix[p.n_dirs] <= 0) return;
  const bool vec = (p.L % R) == 0;
  const bool mask = p.L != R * kWave;
  if constexpr (R > 1) {
    if (!vec) {
      launch_vm<R, false, true>(p, jacobi, st);
      return;
    }
  }
  if (mask)
    launch_vm<R, true, true>(p, jacobi, st);
  else
    launch_vm<R, true, false>(p, jacobi, st);
}

template void launch_sweep_bwd<MPL_INST_R>(const BackParams&, bool, hipStream_t);

}  // namespace mpl
