// Forward scan of TRWP / ISGMR for gfx950: one wavefront per chain, see mp_common.h.
//
// Per pixel p of a chain (front pixel q = p - step), following HorizontalKernel /
// DiagonalKernelWide / DiagonalKernelNarrow of the reference (TRWP_forward.cu:82-376,
// ISGMR_forward.cu:123-431):
//     a[fd]  = U[q, fd] + rho * m[q, fd]                  (m[q] = message just computed, 0 at the start)
//     v[cd]  = min_fd a[fd] + w[p] * ctx(cd, fd)          (largest fd on ties)
//     m[p,:] = v - min_cd v                               (largest cd on ties)
// with U = rho * (S - m_dir_old) - m_inv_old taken from the belief plane S = unary + sum_k m_k
// instead of re-summing all messages (UpdateUnaryKernel, TRWP_forward.cu:60-80).  TRWP (Gauss-Seidel
// over directions) forms U on the fly from S, m_dir, m_inv and keeps S up to date; ISGMR (Jacobi)
// finds U of every direction precomputed in place of the old messages.
//
// Compiled once per R (labels per lane) and per kind of scan (with or without argmin labels) with
// -DMPL_INST_R=<R> -DMPL_INST_TRAIN=<0|1>.

#include <type_traits>

#include "mp_common.h"

namespace mpl {
namespace {

template <int R>
struct PixF {
  float s[R], md[R], mi[R];
  float w;
};

// Dense O(L^2) step: v[cd] = min_fd( a[fd] + w * ctx(cd, fd) ), largest fd on ties.
// HorizontalKernel inner loop, TRWP_forward.cu:127-153.  a_s / ctx_s live in LDS.
template <int R, bool TRAIN>
__device__ __forceinline__ void dense_step(const float (&a)[R], const bool (&valid)[R], float w,
                                           int L, int ctx2d, int lab0, float* a_s,
                                           const float* ctx_s, float (&v)[R], int (&fd_idx)[R]) {
#pragma unroll
  for (int j = 0; j < R; ++j)
    if (valid[j]) a_s[lab0 + j] = a[j];
  __syncthreads();
  int labc[R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    int l = lab0 + j;
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
      if (TRAIN) {
        bool take = (fd == L - 1) || (val < v[j]);
        v[j] = take ? val : v[j];
        fd_idx[j] = take ? fd : fd_idx[j];
      } else {
        v[j] = fminf(v[j], val);
      }
    }
  }
  __syncthreads();
}

// Dense O(L^2) step for 1-D contexts and several labels per lane.  The front labels are visited
// in ascending order; the context values c[|cd - fd|] of the lane's labels are kept in registers and
// moved one label up per front label (c[|cd - (fd+1)|] of label cd is c[|(cd-1) - fd|] of label
// cd - 1; c[fd+1] enters at label 0) with one lane shift.  Both a[fd] and the entering c[fd+1] are
// the same for every lane: they are read from LDS, every lane from the same address (a_w: this
// wavefront's own copy of a[], written at the start of the step; c1_s: the table moved down by one
// entry, c1_s[i] = c[i+1]), four front labels per read, one trip of T = 4 R front labels ahead of
// their use, so the loop waits for none of them.  The shift writes into the register the read
// filled (lane 0 has no source lane and keeps c[fd+1]): no instruction sets up a fill.
// Two front labels are folded per minimum (v_min3).
// TRAIN: the argmin label is found in two steps.  The scan only notes, per label, the trip whose
// candidates last reached the running minimum (the minimum over a trip's candidates against the
// minimum so far, `<=`: one comparison and one select per trip instead of one per front label), and
// returns that trip's first front label in `trip0`; dense1d_argmin then evaluates the T candidates
// of that one trip again.  The argmin the reference keeps is the largest front label whose candidate
// equals the final minimum (its descending scan with `<`): it lies in the last trip that holds such
// a candidate, and that is the last trip whose own minimum is <= the minimum before it.
// The scan covers the front labels fd_lo .. fd_hi - 1 (fd_lo a multiple of T): all of them, or the
// share of one wavefront where several scan a pixel together (split_combine below).  cv0: the
// sliding values at fd_lo, c[|cd - fd_lo|].
template <int R>
constexpr int dense_trip() { return 4 * R; }

template <int R, bool TRAIN>
__device__ __forceinline__ void dense1d_step(const float (&a)[R], const float w, const int lab0,
                                             float* a_w, const float* c1_s, const float (&cv0)[R],
                                             float (&v)[R], int (&trip0)[R], const int fd_lo,
                                             const int fd_hi) {
  constexpr int T = dense_trip<R>();
  float cv[R];
  int rel[R];  // the noted trip, counted back from the current one (0, -1, ...)
#pragma unroll
  for (int j = 0; j < R; ++j) {
    a_w[lab0 + j] = a[j];
    cv[j] = cv0[j];
    v[j] = INFINITY;
    rel[j] = 0;
  }
  auto shift = [&](const float fill) __attribute__((always_inline)) {
    const float in0 = wave_shr1(cv[R - 1], fill);
#pragma unroll
    for (int j = R - 1; j > 0; --j) cv[j] = cv[j - 1];
    cv[0] = in0;
  };
  // the end of a trip: fold its minimum into the running one and note the trip where it reaches it
  auto close_trip = [&](const float (&lm)[R]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const bool take = lm[j] <= v[j];
      v[j] = fminf(v[j], lm[j]);
      rel[j] = take ? 0 : rel[j] - 1;
    }
  };
  float ba[T], bc[T];  // a[fd0 + u], c[fd0 + u + 1]
  auto read4 = [&](const float* src, float (&dst)[T], const int q) __attribute__((always_inline)) {
    const f32x4 x = *reinterpret_cast<const f32x4*>(src + 4 * q);
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[4 * q + i] = x[i];
  };
  // The register a read of c fills becomes a sliding value and stays one for R shifts: the four of
  // group q are free again after shift 4 q + 3 + R of a trip, and that is where the group's next
  // read stands -- in the same trip for the trip after it (kNext groups), or, for the last groups,
  // at the start of the trip that uses them.
  constexpr int kNext = (T - 3 - R + 3) / 4;  // groups q with 4 q + 3 + R < T
  int fd0 = fd_lo;
#pragma unroll
  for (int q = 0; q < R; ++q) read4(a_w + fd0, ba, q);
#pragma unroll
  for (int q = 0; q < kNext; ++q) read4(c1_s + fd0, bc, q);
  for (; fd0 + T <= fd_hi; fd0 += T) {
    float lm[R];  // TRAIN: the minimum over this trip's candidates
#pragma unroll
    for (int u = 0; u < T; u += 2) {
      float v0[R], v1[R];
#pragma unroll
      for (int j = 0; j < R; ++j) v0[j] = fmaf(w, cv[j], ba[u]);
      shift(bc[u]);
#pragma unroll
      for (int j = 0; j < R; ++j) v1[j] = fmaf(w, cv[j], ba[u + 1]);
      shift(bc[u + 1]);
#pragma unroll
      for (int j = 0; j < R; ++j) {
        if (TRAIN)
          lm[j] = u == 0 ? fminf(v0[j], v1[j]) : fminf(fminf(lm[j], v0[j]), v1[j]);
        else
          v[j] = fminf(fminf(v[j], v0[j]), v1[j]);
      }
      // reads that stand after the shifts u and u + 1
#pragma unroll
      for (int s = u; s < u + 2; ++s) {
        if ((s & 3) == 3) read4(a_w + fd0 + T, ba, s / 4);  // a: free once its four labels are done
        if (s >= 3 + R && ((s - 3 - R) & 3) == 0) read4(c1_s + fd0 + T, bc, (s - 3 - R) / 4);
        if (s + T >= 3 + R && s + T - 3 - R < T && ((s + T - 3 - R) & 3) == 0 &&
            (s + T - 3 - R) / 4 >= kNext)
          read4(c1_s + fd0, bc, (s + T - 3 - R) / 4);
      }
    }
    if (TRAIN) close_trip(lm);
  }
  // what is left of the share: fewer than T front labels, one at a time
  if (fd0 < fd_hi) {
#pragma unroll
    for (int q = kNext; q < R; ++q) read4(c1_s + fd0, bc, q);
    float lm[R];
#pragma unroll
    for (int j = 0; j < R; ++j) lm[j] = INFINITY;
#pragma unroll
    for (int u = 0; u < T - 1; ++u) {
      if (fd0 + u < fd_hi) {  // wave-uniform
#pragma unroll
        for (int j = 0; j < R; ++j) {
          const float val = fmaf(w, cv[j], ba[u]);
          if (TRAIN)
            lm[j] = fminf(lm[j], val);
          else
            v[j] = fminf(v[j], val);
        }
        shift(bc[u]);
      }
    }
    if (TRAIN) close_trip(lm);
    fd0 += T;
  }
#pragma unroll
  for (int j = 0; j < R; ++j) trip0[j] = (fd0 - T) + rel[j] * T;
}

// The argmin labels of dense1d_step: for every label of the lane, the largest front label of the
// trip starting at trip0 whose candidate a[fd] + w * c[|cd - fd|] equals the minimum v (the same
// multiply-add on the same operands as in the scan: the same bits).  a_w: the wavefront's copy of
// a[] (front labels past the last one read as +inf or as whatever lies there: their candidates
// are not the minimum); csym_s: the table laid out around its centre, csym_s[dense_sym_centre<R>() + d]
// = c[|d|], so that a lane reads the entries of consecutive front labels at consecutive addresses.
template <int R>
constexpr int dense_sym_centre() { return R * kWave; }  // |cd - fd| < R * 64

template <int R>
__device__ __forceinline__ void fill_dense_sym(float* csym_s, const float* ctx, int L, int tid,
                                               int n_threads) {
  for (int i = tid; i < dense_sym_floats(R); i += n_threads) {
    const int d = i < dense_sym_centre<R>() ? dense_sym_centre<R>() - i : i - dense_sym_centre<R>();
    csym_s[i] = d < L ? ctx[d] : 0.f;
  }
}

template <int R>
__device__ __forceinline__ void dense1d_argmin(const float (&v)[R], const int (&trip0)[R],
                                               const float w, const int lab0, const int L,
                                               const float* a_w, const float* csym_s,
                                               int (&fd_idx)[R]) {
  constexpr int T = dense_trip<R>();
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int t0 = trip0[j];
    const int l = lab0 + j < L ? lab0 + j : L - 1;
    float af[T];
#pragma unroll
    for (int q = 0; q < T / 4; ++q) {
      const f32x4 x = *reinterpret_cast<const f32x4*>(a_w + t0 + 4 * q);
#pragma unroll
      for (int i = 0; i < 4; ++i) af[4 * q + i] = x[i];
    }
    const float* cp = csym_s + (dense_sym_centre<R>() + l - t0 - (T - 1));  // entry of front label t0 + T - 1
    int arg = 0;
#pragma unroll
    for (int u = 0; u < T; ++u) {
      const float val = fmaf(w, cp[T - 1 - u], af[u]);
      arg = val == v[j] ? u : arg;
    }
    const int fd = t0 + arg;
    fd_idx[j] = fd < L ? fd : L - 1;  // (only where no candidate is finite)
  }
}

// The same scan with both broadcasts taken from the lanes that hold the values (v_readlane of a[]
// and of the lane's own table entries c[label]) instead of LDS: no staging, no reads in flight, and
// little state outside the step.  Two more issue slots per front label than dense1d_step; it is the
// step that a kernel compiled for a band or a truncated-linear table takes at a pixel with a
// negative edge weight, where the band and the label scans do not hold.
// `<=` on the ascending scan keeps the largest front label among equals, as the reference's
// descending scan with `<` does.  fd_lo a multiple of R.
template <int R, bool TRAIN, bool WHOLE>  // WHOLE: L is a multiple of R
__device__ __forceinline__ void dense1d_step_lanes(const float (&a)[R], float w, int L, int lab0,
                                             const float* ctx_s, float (&v)[R], int (&fd_idx)[R],
                                             const int fd_lo, const int fd_hi) {
  float c_own[R], cv[R];  // c[label] of the lane's labels; the sliding c[|label - fd|]
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int l = lab0 + j < L ? lab0 + j : L - 1;
    c_own[j] = ctx_s[l];
    cv[j] = fd_lo == 0 ? c_own[j] : ctx_s[l > fd_lo ? l - fd_lo : fd_lo - l];
    v[j] = INFINITY;
    fd_idx[j] = L - 1;
  }
  // the weight in a vector register: a multiply-add takes one scalar operand, and that is a[fd]
  float wv = w;
  asm volatile("" : "+v"(wv));
  // one front label: fd = fd0 + u is owned by lane src = fd0 / R, register u
  auto visit = [&](const int fd, const int u, const int src) __attribute__((always_inline)) {
    const float af = readlane_f(a[u], src);
    // c[fd + 1]: the next label's own entry (past the last label the value is never used)
    const float cn = u + 1 < R ? readlane_f(c_own[u + 1 < R ? u + 1 : 0], src)
                               : readlane_f(c_own[0], (src + 1) & 63);
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const float val = fmaf(wv, cv[j], af);
      if (TRAIN) {
        // (the minimum and the comparison are independent instructions; a select of the value
        // would wait for the comparison's lane mask like the select of the label does)
        const bool take = val <= v[j];
        v[j] = fminf(v[j], val);
        fd_idx[j] = take ? fd : fd_idx[j];
      } else {
        v[j] = fminf(v[j], val);
      }
    }
    const float in0 = wave_shr1(cv[R - 1], cn);
#pragma unroll
    for (int j = R - 1; j > 0; --j) cv[j] = cv[j - 1];
    cv[0] = in0;
  };
  // Two rounds of R front labels per trip: after R one-label shifts the sliding values sit in
  // registers the shifts created, after 2 R they can be back in the ones the trip started with,
  // so the loop carries no register moves.
  int fd0 = fd_lo;
  int src0 = fd_lo / R;  // the lane that owns front label fd0 (counted along: no division per trip)
  for (; fd0 + 2 * R <= fd_hi; fd0 += 2 * R, src0 += 2) {
#pragma unroll
    for (int u = 0; u < 2 * R; ++u) visit(fd0 + u, u % R, src0 + u / R);
  }
  for (; fd0 < fd_hi; fd0 += R, ++src0) {
#pragma unroll
    for (int u = 0; u < R; ++u)
      if (WHOLE || fd0 + u < fd_hi) visit(fd0 + u, u, src0);  // wave-uniform
  }
}

// Several wavefronts on one chain (launches with far fewer chains than the chip has SIMDs, dense
// table): every wavefront of the workgroup walks the chain and holds the same state, but scans only
// its share of the front labels of a pixel; the partial minima (and their labels) meet in LDS,
// one slot per wavefront, and every wavefront folds all of them in the order of the front labels
// (`<=`: the later share wins ties, as the one scan over all front labels does), so the state stays
// identical in all of them, bit for bit what one wavefront computes.  Two sets of slots alternate:
// a wavefront that runs ahead writes the other set, and it cannot reach this set again before the
// barrier of the next step, which every wavefront passes only after it has read this one.
template <int R, bool TRAIN>
__device__ __forceinline__ void split_combine(float* xchg, int n_waves, int wave, int lane, int parity,
                                              float (&v)[R], int (&fd_idx)[R]) {
  constexpr int S = TRAIN ? 2 * R : R;  // dwords per lane and slot
  float* set = xchg + (size_t)parity * n_waves * kWave * S;
  float* mine = set + ((size_t)wave * kWave + lane) * S;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    mine[j] = v[j];
    if (TRAIN) mine[R + j] = __builtin_bit_cast(float, fd_idx[j]);
  }
  __syncthreads();
  for (int k = 0; k < n_waves; ++k) {
    const float* theirs = set + ((size_t)k * kWave + lane) * S;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const float pv = theirs[j];
      if (TRAIN) {
        const int pi = __builtin_bit_cast(int, theirs[R + j]);
        const bool take = (k == 0) || (pv <= v[j]);
        v[j] = take ? pv : v[j];
        fd_idx[j] = take ? pi : fd_idx[j];
      } else {
        v[j] = k == 0 ? pv : fminf(v[j], pv);
      }
    }
  }
}

// Dense step for L <= 64 (one label per lane): a[fd] is broadcast with v_readlane and the context
// comes from a full table tab[fd * L + cd] in LDS, which consecutive lanes read without bank
// conflicts.  Same scan order as dense_step.
template <bool TRAIN>
__device__ __forceinline__ void dense_step_r1(float a, int L, float w, int lane, const float* tab,
                                              float& v, int& fd_idx) {
  const float* col = tab + (lane < L ? lane : L - 1);
  float best = INFINITY;
  int arg = L - 1;
#pragma unroll 4
  for (int fd = L - 1; fd >= 0; --fd) {
    const float af = readlane_f(a, fd);
    const float val = fmaf(w, col[fd * L], af);
    if (TRAIN) {
      const bool take = (fd == L - 1) || (val < best);
      best = take ? val : best;
      arg = take ? fd : arg;
    } else {
      best = fminf(best, val);
    }
  }
  v = best;
  fd_idx = arg;
}

// For the 21 candidates of a lane's label and their minimum `best`: the largest fd with
// val[fd] == best, and in `red` (on entry: best in the lanes of the 21 labels, +inf elsewhere) the
// minimum over lanes 0..31 in lane 31.
// A comparison leaves its lane mask in scalar registers, and a select may read such a mask only two
// issue slots after it was written; a lane shift may read a vector register only two slots after
// it was written.  The compiler keeps every mask in vcc and pads each of these pairs with idle
// slots (some 50 per pixel, and a wavefront that has its SIMD to itself pays for every slot), so
// the three chains are interleaved by hand: masks rotate over three registers, every select comes
// at least two instructions after its comparison, every shift at least two after the one before,
// and the first shift three after the start (the compiler wrote `red` just before).
__device__ __forceinline__ void argmin_and_lane_min_21(const float (&val)[21], float best, float& red,
                                                       int& arg) {
  unsigned long long m1, m2;
  asm(
      "v_cmp_eq_f32_e64 vcc, %5, %4\n\t"
      "v_cmp_eq_f32_e64 %2, %6, %4\n\t"
      "v_cmp_eq_f32_e64 %3, %7, %4\n\t"
      "v_min_f32_dpp %1, %1, %1 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_cndmask_b32_e64 %0, 20, 0, vcc\n\t"
      "v_cmp_eq_f32_e64 vcc, %8, %4\n\t"
      "v_min_f32_dpp %1, %1, %1 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
      "v_cndmask_b32_e64 %0, %0, 1, %2\n\t"
      "v_cmp_eq_f32_e64 %2, %9, %4\n\t"
      "v_min_f32_dpp %1, %1, %1 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
      "v_cndmask_b32_e64 %0, %0, 2, %3\n\t"
      "v_cmp_eq_f32_e64 %3, %10, %4\n\t"
      "v_min_f32_dpp %1, %1, %1 row_shr:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_cndmask_b32_e64 %0, %0, 3, vcc\n\t"
      "v_cmp_eq_f32_e64 vcc, %11, %4\n\t"
      "v_min_f32_dpp %1, %1, %1 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "v_cndmask_b32_e64 %0, %0, 4, %2\n\t"
      "v_cmp_eq_f32_e64 %2, %12, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 5, %3\n\t"
      "v_cmp_eq_f32_e64 %3, %13, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 6, vcc\n\t"
      "v_cmp_eq_f32_e64 vcc, %14, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 7, %2\n\t"
      "v_cmp_eq_f32_e64 %2, %15, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 8, %3\n\t"
      "v_cmp_eq_f32_e64 %3, %16, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 9, vcc\n\t"
      "v_cmp_eq_f32_e64 vcc, %17, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 10, %2\n\t"
      "v_cmp_eq_f32_e64 %2, %18, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 11, %3\n\t"
      "v_cmp_eq_f32_e64 %3, %19, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 12, vcc\n\t"
      "v_cmp_eq_f32_e64 vcc, %20, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 13, %2\n\t"
      "v_cmp_eq_f32_e64 %2, %21, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 14, %3\n\t"
      "v_cmp_eq_f32_e64 %3, %22, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 15, vcc\n\t"
      "v_cmp_eq_f32_e64 vcc, %23, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 16, %2\n\t"
      "v_cmp_eq_f32_e64 %2, %24, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 17, %3\n\t"
      "v_cmp_eq_f32_e64 %3, %25, %4\n\t"
      "v_cndmask_b32_e64 %0, %0, 18, vcc\n\t"
      "v_cndmask_b32_e64 %0, %0, 19, %2\n\t"
      "v_cndmask_b32_e64 %0, %0, 20, %3\n\t"
      : "=&v"(arg), "+v"(red), "=&s"(m1), "=&s"(m2)
      : "v"(best), "v"(val[0]), "v"(val[1]), "v"(val[2]), "v"(val[3]), "v"(val[4]), "v"(val[5]), "v"(val[6]), "v"(val[7]), "v"(val[8]), "v"(val[9]), "v"(val[10]), "v"(val[11]), "v"(val[12]), "v"(val[13]), "v"(val[14]), "v"(val[15]), "v"(val[16]), "v"(val[17]), "v"(val[18]), "v"(val[19]), "v"(val[20])
      : "vcc");
}

// Several labels per lane, no argmin labels: the wavefront minimum of the beliefs and, in the issue
// slots its six lane-shift minima leave (a lane shift may read a register two slots after it was
// written, and a wavefront that has its SIMD to itself pays for every idle slot), the centre tap and
// the first tap of the band step: on exit v[j] = min(a[j] + w c[0], min(a[label-1], a[label+1]) + w c[1]),
// up / dn hold the beliefs of the labels one up and one down, and `red` holds in lane 63 the minimum
// of a[] over the wavefront.  The same operations on the same operands as wave_min_fast and
// band_step's first tap: the same bits.  w: the edge weight in a vector register.
#define MPL_RED(CTRL) "v_min_f32_dpp %0, %0, %0 " CTRL " bank_mask:0xf\n\t"
__device__ __forceinline__ void band_head(const float (&a)[2], float w, float c0, float c1, float& red,
                                          float (&v)[2], float (&up)[2], float (&dn)[2]) {
  float tu, td, q0, q1, p0, p1;
  red = fminf(a[0], a[1]);
  asm("v_mov_b32 %1, 0x7f800000\n\t"
      "v_mov_b32 %2, 0x7f800000\n\t"
      MPL_RED("row_shr:1 row_mask:0xf")
      "v_fma_f32 %5, %9, %10, %7\n\t"
      "v_fma_f32 %6, %9, %10, %8\n\t"
      MPL_RED("row_shr:2 row_mask:0xf")
      "v_mov_b32_dpp %1, %7 wave_shl:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_mov_b32_dpp %2, %8 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
      MPL_RED("row_shr:4 row_mask:0xf")
      "v_min_f32 %3, %8, %2\n\t"
      "v_min_f32 %4, %1, %7\n\t"
      MPL_RED("row_shr:8 row_mask:0xf")
      "v_fmac_f32 %3, %9, %11\n\t"
      "v_fmac_f32 %4, %9, %11\n\t"
      MPL_RED("row_bcast:15 row_mask:0xa")
      "v_min_f32 %5, %5, %3\n\t"
      "v_min_f32 %6, %6, %4\n\t"
      "v_min_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf"
      : "+v"(red), "=&v"(tu), "=&v"(td), "=&v"(q0), "=&v"(q1), "=&v"(p0), "=&v"(p1)
      : "v"(a[0]), "v"(a[1]), "v"(w), "v"(c0), "v"(c1));
  v[0] = p0;
  v[1] = p1;
  up[0] = a[1];
  up[1] = tu;
  dn[0] = td;
  dn[1] = a[0];
}

__device__ __forceinline__ void band_head(const float (&a)[3], float w, float c0, float c1, float& red,
                                          float (&v)[3], float (&up)[3], float (&dn)[3]) {
  float tu, td, q0, q1, q2, p0, p1, p2;
  red = fminf(fminf(a[0], a[1]), a[2]);
  // %0 red  %1 tu  %2 td  %3..%5 q  %6..%8 p  %9..%11 a  %12 w  %13 c0  %14 c1
  asm("v_mov_b32 %1, 0x7f800000\n\t"
      "v_mov_b32 %2, 0x7f800000\n\t"
      MPL_RED("row_shr:1 row_mask:0xf")
      "v_fma_f32 %6, %12, %13, %9\n\t"
      "v_fma_f32 %7, %12, %13, %10\n\t"
      MPL_RED("row_shr:2 row_mask:0xf")
      "v_mov_b32_dpp %1, %9 wave_shl:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_mov_b32_dpp %2, %11 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
      MPL_RED("row_shr:4 row_mask:0xf")
      "v_fma_f32 %8, %12, %13, %11\n\t"
      "v_min_f32 %4, %11, %9\n\t"
      MPL_RED("row_shr:8 row_mask:0xf")
      "v_min_f32 %3, %10, %2\n\t"
      "v_min_f32 %5, %1, %10\n\t"
      MPL_RED("row_bcast:15 row_mask:0xa")
      "v_fmac_f32 %3, %12, %14\n\t"
      "v_fmac_f32 %4, %12, %14\n\t"
      MPL_RED("row_bcast:31 row_mask:0xc")
      "v_fmac_f32 %5, %12, %14\n\t"
      "v_min_f32 %6, %6, %3\n\t"
      "v_min_f32 %7, %7, %4\n\t"
      "v_min_f32 %8, %8, %5"
      : "+v"(red), "=&v"(tu), "=&v"(td), "=&v"(q0), "=&v"(q1), "=&v"(q2), "=&v"(p0), "=&v"(p1),
        "=&v"(p2)
      : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(w), "v"(c0), "v"(c1));
  v[0] = p0;
  v[1] = p1;
  v[2] = p2;
  up[0] = a[1];
  up[1] = a[2];
  up[2] = tu;
  dn[0] = td;
  dn[1] = a[0];
  dn[2] = a[1];
}

__device__ __forceinline__ void band_head(const float (&a)[4], float w, float c0, float c1, float& red,
                                          float (&v)[4], float (&up)[4], float (&dn)[4]) {
  float tu, td, q0, q1, q2, q3, p0, p1, p2, p3;
  red = fminf(fminf(a[0], a[1]), fminf(a[2], a[3]));
  // %0 red  %1 tu  %2 td  %3..%6 q  %7..%10 p  %11..%14 a  %15 w  %16 c0  %17 c1
  asm("v_mov_b32 %1, 0x7f800000\n\t"
      "v_mov_b32 %2, 0x7f800000\n\t"
      MPL_RED("row_shr:1 row_mask:0xf")
      "v_fma_f32 %7, %15, %16, %11\n\t"
      "v_fma_f32 %8, %15, %16, %12\n\t"
      MPL_RED("row_shr:2 row_mask:0xf")
      "v_mov_b32_dpp %1, %11 wave_shl:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_mov_b32_dpp %2, %14 wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
      MPL_RED("row_shr:4 row_mask:0xf")
      "v_fma_f32 %9, %15, %16, %13\n\t"
      "v_fma_f32 %10, %15, %16, %14\n\t"
      MPL_RED("row_shr:8 row_mask:0xf")
      "v_min_f32 %4, %13, %11\n\t"
      "v_min_f32 %5, %14, %12\n\t"
      MPL_RED("row_bcast:15 row_mask:0xa")
      "v_min_f32 %3, %12, %2\n\t"
      "v_min_f32 %6, %1, %13\n\t"
      MPL_RED("row_bcast:31 row_mask:0xc")
      "v_fmac_f32 %3, %15, %17\n\t"
      "v_fmac_f32 %4, %15, %17\n\t"
      "v_fmac_f32 %5, %15, %17\n\t"
      "v_fmac_f32 %6, %15, %17\n\t"
      "v_min_f32 %7, %7, %3\n\t"
      "v_min_f32 %8, %8, %4\n\t"
      "v_min_f32 %9, %9, %5\n\t"
      "v_min_f32 %10, %10, %6"
      : "+v"(red), "=&v"(tu), "=&v"(td), "=&v"(q0), "=&v"(q1), "=&v"(q2), "=&v"(q3), "=&v"(p0),
        "=&v"(p1), "=&v"(p2), "=&v"(p3)
      : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(w), "v"(c0), "v"(c1));
  v[0] = p0;
  v[1] = p1;
  v[2] = p2;
  v[3] = p3;
  up[0] = a[1];
  up[1] = a[2];
  up[2] = a[3];
  up[3] = tu;
  dn[0] = td;
  dn[1] = a[0];
  dn[2] = a[1];
  dn[3] = a[2];
}
#undef MPL_RED
// Band O(L*K) step for 1-D contexts with a constant tail (c[k] == cmax for k >= K, c[k] <= cmax
// below), exact for w >= 0:
//   v[cd] = min( min_{|k|<K} a[cd+k] + w*c[|k|],  min_fd a[fd] + w*cmax )
// The second term is an upper bound for every label and is attained by all labels farther than the
// band from argmin(a); fp32 addition is monotone, so the values are bit-identical to the dense scan.
// KT > 0: KT - 1 taps with c[] in registers (KT >= K).  KT == 0: K at run time, taps in LDS.
// HEAD (band_head ran: KT >= 2 in registers, several labels per lane, no argmin labels): v, up and dn come in as the
// first tap left them, and the taps go on from the second.
template <int R, bool TRAIN, int KT, bool HEAD = false>
__device__ __forceinline__ void band_step(const float (&a)[R], float w, int K, const float* c_reg,
                                          const float* ctx_s, float cmax, float amin, int fstar,
                                          int lab0, float (&v)[R], int (&fd_idx)[R],
                                          const float* up_in = nullptr, const float* dn_in = nullptr) {
  static_assert(!HEAD || (KT >= 2 && !TRAIN), "the head covers the first tap of a band in registers");
  const float inf = INFINITY;
  float up[R], dn[R];
  int off[R];
  const float c0 = KT > 0 ? c_reg[0] : ctx_s[0];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    up[j] = HEAD ? up_in[j] : a[j];
    dn[j] = HEAD ? dn_in[j] : a[j];
    if (!HEAD) v[j] = fmaf(w, c0, a[j]);
    off[j] = 0;
  }
  // `refill`: up[0] / dn[R-1] still hold unshifted beliefs, so the vacated lane is set to +inf;
  // from tap R+1 on every vector has been through one such shift and the lane keeps its +inf
  auto tap = [&](int k, float ck, bool refill) {
    // one-label shifts: up[j] <- a[label + k], dn[j] <- a[label - k]
    float tu = refill ? wave_shl1(up[0], inf) : wave_shl1_keep(up[0]);
    float td = refill ? wave_shr1(dn[R - 1], inf) : wave_shr1_keep(dn[R - 1]);
#pragma unroll
    for (int j = 0; j < R - 1; ++j) up[j] = up[j + 1];
    up[R - 1] = tu;
#pragma unroll
    for (int j = R - 1; j > 0; --j) dn[j] = dn[j - 1];
    dn[0] = td;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      if (TRAIN) {
        float cu = fmaf(w, ck, up[j]);
        float cd = fmaf(w, ck, dn[j]);
        bool tk = cu <= v[j];  // larger front label wins ties
        v[j] = tk ? cu : v[j];
        off[j] = tk ? k : off[j];
        bool tk2 = cd < v[j];  // smaller front label loses ties
        v[j] = tk2 ? cd : v[j];
        off[j] = tk2 ? -k : off[j];
      } else {
        // x -> fma(w, ck, x) is monotone, so the smaller belief of the two gives the smaller
        // candidate: one multiply-add per tap and label, the same bits
        v[j] = fminf(v[j], fmaf(w, ck, fminf(up[j], dn[j])));
      }
    }
  };
  if (KT > 0) {
#pragma unroll
    for (int k = HEAD ? 2 : 1; k < KT; ++k) tap(k, c_reg[k], k <= R);
  } else {
    // R taps per trip: the R one-label rotations of up[] / dn[] then cancel, so the loop carries
    // no register moves, and the R coefficients are fetched from LDS together
    int k = 1;
    if (K > R) {
      float cc[R];
#pragma unroll
      for (int u = 0; u < R; ++u) cc[u] = ctx_s[1 + u];
#pragma unroll
      for (int u = 0; u < R; ++u) tap(1 + u, cc[u], true);
      k = 1 + R;
      for (; k + R <= K; k += R) {
#pragma unroll
        for (int u = 0; u < R; ++u) cc[u] = ctx_s[k + u];
#pragma unroll
        for (int u = 0; u < R; ++u) tap(k + u, cc[u], false);
      }
#pragma unroll
      for (int u = 0; u < R - 1; ++u)
        if (k + u < K) tap(k + u, ctx_s[k + u], false);
    } else {
#pragma unroll
      for (int u = 0; u < R - 1; ++u)
        if (1 + u < K) tap(1 + u, ctx_s[1 + u], true);
    }
  }
  const float far = fmaf(w, cmax, amin);
#pragma unroll
  for (int j = 0; j < R; ++j) {
    if (TRAIN) {
      int fb = lab0 + j + off[j];
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

// O(L log L / 64) step for truncated linear contexts c[k] = min(s*k, cmax) of any width, w >= 0.
// With t = w*s,
//   min_{fd <= cd} a[fd] + t*(cd - fd) =  t*cd + prefixmin_{fd <= cd} (a[fd] - t*fd)
//   min_{fd >= cd} a[fd] + t*(fd - cd) = -t*cd + suffixmin_{fd >= cd} (a[fd] + t*fd)
// so two scans over the labels find, for every cd, the best front label on either side; a label
// beyond the truncation can only win where the far candidate min(a) + w*cmax is at least as good.
// The scans run on rounded differences, so they only *select* the candidates (the largest label
// among equals on each side, as the reference's scan order does); the values are then evaluated
// from the table exactly as the dense scan does, a[fd] + w*c[|cd - fd|], and compared with the far
// candidate.  A selection off by the rounding of t*L picks a value within a few ulp of the largest
// belief of the true minimum.
template <int R, bool TRAIN>
__device__ __forceinline__ void linear_step(const float (&a)[R], float w, float slope, float cmax,
                                            float amin, int fstar, int lab0, int lane, int L,
                                            float* a_s, const float* ctx_s, float (&v)[R],
                                            int (&fd_idx)[R]) {
  const float inf = INFINITY;
  constexpr int big = 0x7fffffff;
  const float t = w * slope;
  float gm[R], gp[R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const float l = (float)(lab0 + j);
    gm[j] = fmaf(-t, l, a[j]);
    gp[j] = fmaf(t, l, a[j]);
    a_s[lab0 + j] = a[j];  // staged for the gathers below
  }
  // left side: prefix minimum and its largest achiever (the largest label up to cd whose own
  // prefix minimum it is)
  float q[R], pl[R];
  q[0] = gm[0];
#pragma unroll
  for (int j = 1; j < R; ++j) q[j] = fminf(q[j - 1], gm[j]);
  const float before = wave_shr1(lane_prefix_min(q[R - 1]), inf);
  int qi[R], il[R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    pl[j] = fminf(before, q[j]);
    const int f = (gm[j] == pl[j]) ? lab0 + j : -1;
    qi[j] = j == 0 ? f : max(qi[j > 0 ? j - 1 : 0], f);
  }
  const int before_i = dpp_i<0x138>(-1, lane_prefix_max(qi[R - 1]));  // lane i <- lane i-1
#pragma unroll
  for (int j = 0; j < R; ++j) il[j] = max(max(before_i, qi[j]), 0);
  // right side: suffix minimum; its largest achiever is where the plateau of that minimum ends
  float sfx[R], pr[R], nx[R];
  sfx[R - 1] = gp[R - 1];
#pragma unroll
  for (int j = R - 2; j >= 0; --j) sfx[j] = fminf(sfx[j + 1], gp[j]);
  const float after = wave_shl1(lane_suffix_min(sfx[0], lane), inf);
#pragma unroll
  for (int j = 0; j < R; ++j) pr[j] = fminf(after, sfx[j]);
#pragma unroll
  for (int j = 0; j < R - 1; ++j) nx[j] = pr[j + 1];
  nx[R - 1] = wave_shl1(pr[0], inf);
  int si[R], ir[R];
#pragma unroll
  for (int j = R - 1; j >= 0; --j) {
    const int b = (pr[j] < nx[j]) ? lab0 + j : big;
    si[j] = j == R - 1 ? b : min(si[j < R - 1 ? j + 1 : j], b);
  }
  const int after_i = dpp_i<0x130>(big, lane_suffix_min(si[0], lane));  // lane i <- lane i+1
#pragma unroll
  for (int j = 0; j < R; ++j) ir[j] = min(min(after_i, si[j]), L - 1);
  __syncthreads();  // a_s
  const float far = fmaf(w, cmax, amin);
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int cd = lab0 + j;
    const int kl = cd - il[j], kr = ir[j] - cd;
    const float vl = fmaf(w, ctx_s[kl < 0 ? 0 : (kl < L ? kl : L - 1)], a_s[il[j]]);
    const float vr = fmaf(w, ctx_s[kr < 0 ? 0 : kr], a_s[ir[j]]);
    const bool tr = vr <= vl;  // the larger front label wins ties
    float best = tr ? vr : vl;
    int arg = tr ? ir[j] : il[j];
    const bool lt = far < best, eq = far == best;
    if (TRAIN) fd_idx[j] = lt ? fstar : (eq ? (arg > fstar ? arg : fstar) : arg);
    v[j] = lt ? far : best;
  }
  __syncthreads();  // the next step overwrites a_s
}

// One chain.  KT: > 0 band with compile-time K, 0 band with run-time K, -1 dense, -21 dense with
// exactly 21 labels, -2 truncated linear context of any width (linear_step), -3 dense 1-D table with
// the front labels split over the wavefronts of the workgroup (split_combine; xchg: its LDS slots).
// VEC: L % R == 0 (vector accesses).  MASK: some lanes own labels >= L.
// C0: the table's entry 0 is its smallest (band steps only; CtxDesc::c0_is_min), which gives the
// normalisation minimum without a second reduction.
template <int R, bool VEC, bool MASK, bool TRAIN, int JACOBI, int KT, bool C0 = false>
__device__ __forceinline__ void run_chain_fwd(const SweepParams& p, const CtxDesc& desc,
                                              const ChainCtx& ch, float* a_s, const float* ctx_s,
                                              const bool skip_s_store_in, float* xchg = nullptr) {
  constexpr bool SPLIT = (KT == -3);
  const int L = p.L;
  // The caller's initial messages turned out to be all zero (the usual case: the reference's
  // callers pass a cleared tensor) and this is a sweep that can profit: S = Q = U = unary, so the
  // unary terms are read in place of the plane, and the even sweep of the first pair has nothing to
  // store (the odd one reads the unary terms again).  Wave-uniform, the same for every chain.
  const bool zfirst = JACOBI != 2 && p.zero_first && desc.msg_nonzero == 0;
  const bool skip_s_store = skip_s_store_in || (!JACOBI && zfirst && (ch.dir & 1) == 0);
  const int64_t HW = (int64_t)p.H * p.W;
  const int64_t P = (int64_t)p.B * HW;
  const int64_t N = P * L;
  const int dir = ch.dir;
  const int64_t img_p = (int64_t)ch.bv * HW;  // first pixel of this batch item
  const int64_t img_e = img_p * L;
  const int vbytes = L * 4;
  // plane bases of this batch item and direction; descriptors are formed per access
  // Jacobi: the plane of this direction in msg_in holds U itself (written by the host's
  // element-wise pass before the sweeps), so one plane is read per pixel instead of three
  // JACOBI == 2 (four directions, rho == 1): no U plane either; U of the pair {dir, dir^1} is the
  // unary plus the old messages of the other pair, read here (three planes in, but the pass that
  // stores U, five planes in and two out per iteration, is not run)
  const int oth = (dir & ~1) ^ 2;  // the even direction of the other pair
  const float* __restrict__ bS =
      (zfirst ? p.belief_zero
              : (JACOBI == 1 ? p.msg_in + (int64_t)(p.u_pair_share ? (dir & ~1) : dir) * p.u_stride
                             : p.belief)) + img_e;
  const float* __restrict__ bMd = p.msg_in + (int64_t)(JACOBI == 2 ? oth : dir) * N + img_e;
  const float* __restrict__ bMi = p.msg_in + (int64_t)(JACOBI == 2 ? oth + 1 : (dir ^ 1)) * N + img_e;
  float* __restrict__ bMo = p.msg_out + (int64_t)dir * N + img_e;
  float* __restrict__ bSo = (JACOBI ? nullptr : p.belief_out + img_e);
  uint8_t* __restrict__ bImin = TRAIN ? p.idx_min + (int64_t)dir * N + img_e : nullptr;
  const int img_bytes_p = (int)(HW * 4 > 0x7fffffff ? 0x7fffffff : HW * 4);
  const rsrc_t dW = make_rsrc(p.edge + (int64_t)dir * P + img_p, img_bytes_p);
  const rsrc_t dInorm = make_rsrc(TRAIN ? p.idx_norm + (int64_t)dir * P + img_p : nullptr,
                                  TRAIN ? (int)HW : 0);
  const float rho = p.rho;
  const float inf = INFINITY;
  const int lane = SPLIT ? (int)(threadIdx.x & (kWave - 1)) : (int)threadIdx.x;
  const int lab0 = R * lane;
  const int foff = lab0 * 4;  // byte offset of this lane's block inside a pixel's float vector
  const int n = ch.n;
  // SPLIT: the wavefronts of the workgroup share the front labels; the first one stores
  const int wave = SPLIT ? uniform_i((int)(threadIdx.x / kWave)) : 0;
  const int n_waves = SPLIT ? (int)(blockDim.x / kWave) : 1;
  const bool store_ok = !SPLIT || wave == 0;
  // front labels per wavefront: whole trips of the dense scan
  // (the division by the number of wavefronts runs on the vector unit: without the explicit
  // read-back the bounds, and with them the loop counter of the scan and every address it forms,
  // would stay in vector registers)
  const int fd_chunk = SPLIT ? uniform_i(split_share(L, R, n_waves)) : L;
  const int fd_lo = SPLIT ? uniform_i(min(wave * fd_chunk, L)) : 0;
  const int fd_hi = SPLIT ? uniform_i(min(fd_lo + fd_chunk, L)) : L;
  // dense scan, several labels per lane: this wavefront's copy of a[], the table moved down by one
  // entry, and the sliding table values of the lane's labels at the first front label
  float* a_w = a_s + (SPLIT ? wave * kMaxL : 0);
  const float* c1_s = ctx_s + dense_c1_offset(L);
  const float* csym_s = c1_s + dense_c1_floats(L);  // the table around its centre (dense1d_argmin)
  // (only where the dense scan is the kernel's step: a kernel compiled for a band or a
  // truncated-linear table meets it at pixels with a negative edge weight and takes
  // dense1d_step_lanes)
  constexpr bool kDenseMain = R > 1 && (KT == -1 || KT == -3);
  float cv0_chain[R];
  if constexpr (kDenseMain) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int l = lab0 + j < L ? lab0 + j : L - 1;
      cv0_chain[j] = ctx_s[l > fd_lo ? l - fd_lo : fd_lo - l];
    }
  }

  bool valid[R];
  // a lane's labels beyond the last one are kept at +inf by a maximum with +inf (-inf for the
  // others, which changes nothing): one instruction in the short encoding, no lane masks to hold
  float floor_l[R];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    valid[j] = MASK ? (lab0 + j < L) : true;
    floor_l[j] = valid[j] ? -INFINITY : INFINITY;
  }

  float c_reg[KT > 0 ? KT : 1];
  if (KT > 0) {
#pragma unroll
    for (int k = 0; k < KT; ++k) c_reg[k] = p.ctx[k];
  }
  // KT == -21: dense path with the label count fixed at 21 (the segmentation case)
  constexpr int LT = (KT == -21) ? 21 : 0;
  float tcol[LT > 0 ? LT : 1];
  if (LT > 0) {
#pragma unroll
    for (int fd = 0; fd < LT; ++fd) tcol[fd] = ctx_s[fd * LT + (lane < LT ? lane : LT - 1)];
  }
  const int K = desc.band_k;
  // (in a vector register for the whole chain: the far candidate multiplies it by the edge weight
  // and adds the minimum, both scalars, and a multiply-add takes one scalar operand)
  float cmax = desc.cmax;
  asm volatile("" : "+v"(cmax));

  // first Gauss-Seidel iteration over all-zero initial messages: the plane of this direction has
  // not been swept yet, and neither has the opposite one when this direction is the even one
  const bool md_zero = !JACOBI && p.first_iter && desc.msg_nonzero == 0;
  const bool mi_zero = md_zero && (dir & 1) == 0;
  // Gauss-Seidel pairs (p.pair_q): between the sweep of an even direction and the sweep of its
  // opposite the belief plane holds Q = S - m_dir - m_inv, which neither sweep changes:
  //   first sweep  (even):  reads S, m_dir, m_inv; stores m_dir' and Q
  //   second sweep (odd):   reads Q and m_inv (= m_even'), not its own old messages:
  //                         S - m_dir = Q + m_inv;  stores m_dir' and S = Q + m_inv + m_dir'
  // (at a chain start, where no message is written, the plane is converted with the old values)
  const bool pair_first = !JACOBI && p.pair_q && (dir & 1) == 0;
  const bool pair_second = !JACOBI && p.pair_q && (dir & 1) == 1;
  // VEC: one descriptor per plane for the whole kernel, covering the batch item's image; a lane
  // reaches its labels of a pixel through its vector offset, and a lane without labels (or a step
  // that must not store) through an offset no descriptor covers.  Nothing but one multiply, one
  // add and one select per pixel is then spent on addressing (descriptors formed per access cost
  // some eight scalar instructions each, which a chain-starved launch -- one wavefront per SIMD,
  // every instruction an issue slot of its own -- cannot hide).  Planes that are not to be read
  // (all-zero initial messages, the odd sweep's own old messages) or stored get an empty descriptor.
  const bool lane_ok = !MASK || lab0 < L;
  const int img_bytes = (int)(unsigned)(HW * L * 4);
  // (VEC and MASK: a lane without labels carries the size of the image in place of its offset, which
  // takes every access of its past the end of every plane without a select per access; the host
  // gives images beyond 2 GiB, where that sum could wrap, to the kernels that form a descriptor per
  // access)
  // (one label per lane: every image goes through these kernels, and the select stays)
  constexpr bool kAddDead = R > 1;
  const unsigned foff_ok = lane_ok ? (unsigned)foff : (unsigned)img_bytes;
  const rsrc_t rS = make_rsrc(bS, img_bytes);
  const rsrc_t rMd0 = make_rsrc(bMd, md_zero ? 0 : img_bytes);  // chain start
  const rsrc_t rMd = make_rsrc(bMd, (md_zero || pair_second) ? 0 : img_bytes);
  const rsrc_t rMi = make_rsrc(bMi, mi_zero ? 0 : img_bytes);
  const rsrc_t rMo = make_rsrc(bMo, img_bytes);
  const rsrc_t rSo = make_rsrc(bSo, (JACOBI || skip_s_store) ? 0 : img_bytes);
  const rsrc_t rImin = make_rsrc(bImin, TRAIN ? (int)(HW * L) : 0);
  // loads of the next pixel; past the end of the chain the last pixel is fetched again
  const int last_p = ch.pix0 + (n - 1) * ch.pstep;
  int ld_p = ch.pix0;
  int ld_t = 0;
  auto load_next = [&](const bool first = false) __attribute__((always_inline)) {
    PixF<R> r;
    // VEC: the prefetch simply runs on past the end of the chain: what lies there is another pixel
    // of the image or outside the descriptors (reads as 0), and no step uses it
    const unsigned pp = (unsigned)uniform_i((VEC || ld_t < n) ? ld_p : last_p);
    const unsigned so = pp * (unsigned)vbytes;
    if constexpr (VEC) {
      const int vo = (int)(kAddDead ? so + foff_ok : (lane_ok ? so + (unsigned)foff : kDeadWide));
      buf_load<R, true>(rS, vo, 0u, r.s);
      if (JACOBI == 0) {
        buf_load<R, true>(first ? rMd0 : rMd, vo, 0u, r.md);
        buf_load<R, true>(rMi, vo, 0u, r.mi);
      } else if (JACOBI == 2) {
        buf_load<R, true>(rMd0, vo, 0u, r.md);
        buf_load<R, true>(rMi, vo, 0u, r.mi);
      }
    } else {
      const int nrec = (int)(so + (unsigned)vbytes);
      buf_load<R, VEC>(make_rsrc(bS, nrec), foff, so, r.s);
      if (JACOBI == 0) {
        // planes that still hold all-zero initial messages are read through an empty descriptor
        buf_load<R, VEC>(make_rsrc(bMd, (md_zero || (pair_second && ld_t > 0)) ? 0 : nrec), foff, so,
                         r.md);
        buf_load<R, VEC>(make_rsrc(bMi, mi_zero ? 0 : nrec), foff, so, r.mi);
      } else if (JACOBI == 2) {
        buf_load<R, VEC>(make_rsrc(bMd, nrec), foff, so, r.md);
        buf_load<R, VEC>(make_rsrc(bMi, nrec), foff, so, r.mi);
      }
    }
    r.w = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dW, (int)(pp * 4u), 0, 0));
    ld_p += ch.pstep;
    ld_t += 1;
    return r;
  };

  // chain start: its front lies outside the image and the reference never writes it.  The Jacobi
  // buffers alternate, so there the start pixel is written with the zeros it keeps in the reference.
  float prev[R], uf[R];
  {
    const PixF<R> p0 = load_next(true);
    MPL_ORDER_LOADS();  // (the chain start's loads stay ahead of the ring's)
    float conv[R];  // the start pixel's belief-plane value in the other representation
#pragma unroll
    for (int j = 0; j < R; ++j) conv[j] = 0.f;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      prev[j] = 0.f;
      float un = JACOBI == 2 ? (p0.s[j] + p0.md[j]) + p0.mi[j] : p0.s[j];
      if (!JACOBI) {
        const float t0 = pair_second ? p0.s[j] + p0.mi[j] : p0.s[j] - p0.md[j];
        un = fmaf(t0, rho, -p0.mi[j]);
        conv[j] = pair_second ? t0 + p0.md[j] : t0 - p0.mi[j];
      }
      uf[j] = valid[j] ? un : inf;
    }
    if constexpr (SPLIT) {
      // the first wavefront is about to overwrite the start pixel's entry of the belief plane, in
      // place: not before every wavefront of the chain has read it
      wait_vmem<0>();
      __syncthreads();
    }
    const unsigned so0 = (unsigned)ch.pix0 * (unsigned)vbytes;
    const int vo0 = (int)((lane_ok && store_ok) ? so0 + (unsigned)foff : kDeadWide);
    const int nrec0 = store_ok ? (int)(so0 + (unsigned)vbytes) : 0;
    if (!JACOBI && p.pair_q && !skip_s_store) {
      if constexpr (VEC)
        buf_store<R, true>(rSo, vo0, 0u, conv);
      else
        buf_store<R, VEC>(make_rsrc(bSo, nrec0), foff, so0, conv);
    }
    if (JACOBI || p.zero_start) {
      float z[R];
#pragma unroll
      for (int j = 0; j < R; ++j) z[j] = 0.f;
      if constexpr (VEC)
        buf_store<R, true>(rMo, vo0, 0u, z);
      else
        buf_store<R, VEC>(make_rsrc(bMo, nrec0), foff, so0, z);
    }
  }

  // memory instructions per step: 1 or 3 label vectors + the weight in, 1-2 label vectors
  // (+ indices) out
  constexpr int kOps = (JACOBI == 1 ? 1 : 3) * vec_ops(R, VEC) + 1 + (JACOBI ? 1 : 2) * vec_ops(R, VEC) +
                       (TRAIN ? byte_ops(R, VEC) + 1 : 0);
  constexpr int D = ring_depth(kOps);
  // Two banks of D pixels in flight: while the steps consume one, the loads of D pixels ahead land
  // in the other, so that after 2 D steps every value sits in the register it started in (with a
  // single bank the loop ends in one register move per value in flight).
  PixF<R> ring[D], ring2[D];
#pragma unroll
  for (int u = 0; u < D; ++u) {
    ring[u] = load_next();
    // keeps the pixels' loads in this order: the compiler's own waits in the loop are sized for
    // the order it sees here, and a later pixel's loads placed first would make them drain the queue
    MPL_ORDER_LOADS();
  }

  int st_p = ch.pix0 + ch.pstep;
  // in_chain: a constant `true` where the caller knows that step t lies inside the chain and that
  // no edge weight of the chain is negative
  auto step = [&](const PixF<R>& px, const int t, const auto in_chain) __attribute__((always_inline)) {
      constexpr bool kPlain = decltype(in_chain)::value;
      // steps past the end compute on stale data and store nothing
      const bool live = kPlain || t < n;
      float tt[R], un[R];
#pragma unroll
      for (int j = 0; j < R; ++j) {
        float x = JACOBI == 2 ? (px.s[j] + px.md[j]) + px.mi[j] : px.s[j];
        if (!JACOBI) {
          // unary + the other directions' messages
          tt[j] = pair_second ? px.s[j] + px.mi[j] : px.s[j] - px.md[j];
          x = fmaf(tt[j], rho, -px.mi[j]);  // UpdateUnaryKernel, TRWP_forward.cu:70-78
        } else {
          tt[j] = 0.f;
        }
        un[j] = MASK ? fmaxf(x, floor_l[j]) : x;
      }
      const float w = uniform_f(px.w);
      float a[R], v[R];
      int fd_idx[R];
#pragma unroll
      for (int j = 0; j < R; ++j) a[j] = fmaf(rho, prev[j], uf[j]);
      // the normalisation minimum of v (every path ends with it or with a cheaper way to it: the
      // usual path then runs through without a flag to test)
      float nmin;
      auto norm_min = [&]() __attribute__((always_inline)) {
        float vm = inf;
#pragma unroll
        for (int j = 0; j < R; ++j) vm = fminf(vm, MASK ? fmaxf(v[j], floor_l[j]) : v[j]);
        return wave_min_fast(vm);
      };
      // (the usual case falls through; the trips of steps that the caller vouches for do not ask)
      if ((KT >= 0 || KT == -2) && (kPlain || __builtin_expect(w >= 0.f, 1))) {
        // (several labels per lane without argmin labels: the reduction and the first tap in one
        // block)
        constexpr bool kHead = R >= 2 && !TRAIN && KT >= 2;
        float amin;
        float hup[R], hdn[R];
        if constexpr (kHead) {
          float red;
          band_head(a, px.w, c_reg[0], c_reg[1], red, v, hup, hdn);
          amin = readlane_f(red, 63);
        } else {
          float am = a[0];
#pragma unroll
          for (int j = 1; j < R; ++j) am = fminf(am, a[j]);
          amin = wave_min_fast(am);
        }
        int fstar = L - 1;
        if (TRAIN) {
          bool pr[R];
#pragma unroll
          for (int j = 0; j < R; ++j) pr[j] = (a[j] == amin);
          fstar = last_label<R>(pr, L - 1);
        }
        if constexpr (KT == -2) {
          linear_step<R, TRAIN>(a, w, desc.slope, cmax, amin, fstar, lab0, lane, L, a_s, ctx_s, v,
                                fd_idx);
        } else {
          // (after the head the weight is taken from the vector register every lane loaded it
          // into: the minimum arrives in a scalar register, and a multiply-add reads one scalar)
          band_step<R, TRAIN, (KT > 0 ? KT : 0), kHead>(a, kHead ? px.w : w, K, c_reg, ctx_s, cmax, amin,
                                                        fstar, lab0, v, fd_idx, hup, hdn);
        }
        if constexpr (KT != -2 && C0) {
          // every candidate is >= amin + w*c[0], which the centre tap of label argmin(a) attains
          nmin = fmaf(kHead ? px.w : w, KT > 0 ? c_reg[0] : ctx_s[0], amin);
        } else {
          nmin = norm_min();
        }
      } else if (R == 1 && KT < 0 && desc.band_k == 0) {  // (the full table is in LDS then)
        if constexpr (LT > 0) {
          // 21 labels: the scan over front labels fully unrolled, context column in registers.
          // The edge weight stays in a vector register (every lane loaded the same one): a[fd]
          // arrives in a scalar register, and a multiply-add takes one scalar operand only.
          float af[LT], val[LT];
#pragma unroll
          for (int fd = 0; fd < LT; ++fd) af[fd] = readlane_f(a[0], fd);
          // (a multiply-add may read a[fd] only two issue slots after it reached its scalar
          // register: all of them first, then the multiply-adds)
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int fd = 0; fd < LT; ++fd) val[fd] = fmaf(px.w, tcol[fd], af[fd]);
          float best = val[LT - 1];
#pragma unroll
          for (int fd = LT - 2; fd >= 1; fd -= 2) best = fminf(fminf(val[fd], val[fd - 1]), best);
          if ((LT & 1) == 0) best = fminf(best, val[0]);
          v[0] = best;
          if (TRAIN) {
            // the scan in descending order with a strict comparison keeps the largest front label
            // that attains the minimum
            float red = valid[0] ? best : inf;
            argmin_and_lane_min_21(val, best, red, fd_idx[0]);
            nmin = readlane_f(red, 31);
          } else {
            fd_idx[0] = LT - 1;
            nmin = norm_min();
          }
        } else {
          dense_step_r1<TRAIN>(a[0], L, w, lane, ctx_s, v[0], fd_idx[0]);
          nmin = norm_min();
        }
      } else if (live) {
        if constexpr (R > 1) {  // (2-D tables exist for one label per lane only)
          if constexpr (kDenseMain) {
            dense1d_step<R, TRAIN>(a, w, lab0, a_w, c1_s, cv0_chain, v, fd_idx, fd_lo, fd_hi);
            if constexpr (SPLIT) split_combine<R, TRAIN>(xchg, n_waves, wave, lane, t & 1, v, fd_idx);
            // (fd_idx holds the first front label of the trip with the argmin; only a wavefront
            // that stores needs the label itself)
            if (TRAIN && store_ok) dense1d_argmin<R>(v, fd_idx, w, lab0, L, a_w, csym_s, fd_idx);
          } else {
            // a pixel with a negative edge weight in a kernel compiled for a band or a
            // truncated-linear table: the same candidates, broadcast from the lanes
            dense1d_step_lanes<R, TRAIN, VEC>(a, w, L, lab0, ctx_s, v, fd_idx, 0, L);
          }
        } else {
          dense_step<R, TRAIN>(a, valid, w, L, p.ctx2d, lab0, a_s, ctx_s, v, fd_idx);
        }
        nmin = norm_min();
      } else {
#pragma unroll
        for (int j = 0; j < R; ++j) {
          v[j] = 0.f;
          fd_idx[j] = 0;
        }
        nmin = 0.f;
      }
      float m[R], sn[R];
#pragma unroll
      for (int j = 0; j < R; ++j) {
        m[j] = v[j] - nmin;  // MsgNormNaive, commonCUDA.cuh:126-128
        sn[j] = pair_first ? tt[j] - px.mi[j] : tt[j] + m[j];
        prev[j] = m[j];  // (a lane without a label keeps a = +inf through uf, whatever prev is)
        uf[j] = un[j];
      }
      const unsigned sp = (unsigned)uniform_i(st_p);
      const unsigned so = sp * (unsigned)vbytes;
      const unsigned sob = sp * (unsigned)L;
      if constexpr (VEC) {
        const bool on = lane_ok && live && store_ok;  // nothing is stored past the end
        const int vo = (int)(kAddDead ? ((live && store_ok) ? so + foff_ok : kDeadWide)
                                      : (on ? so + (unsigned)foff : kDeadWide));
        buf_store<R, true>(rMo, vo, 0u, m);
        if (!JACOBI) buf_store<R, true>(rSo, vo, 0u, sn);
        if (TRAIN) buf_store_u8<R, true>(rImin, (int)(on ? sob + (unsigned)lab0 : kDeadWide), 0u, fd_idx);
      } else {
        const int nrec = (live && store_ok) ? (int)(so + (unsigned)vbytes) : 0;
        buf_store<R, VEC>(make_rsrc(bMo, nrec), foff, so, m);
        if (!JACOBI) buf_store<R, VEC>(make_rsrc(bSo, skip_s_store ? 0 : nrec), foff, so, sn);
        if (TRAIN)
          buf_store_u8<R, VEC>(make_rsrc(bImin, (live && store_ok) ? (int)(sob + (unsigned)L) : 0), lab0, sob, fd_idx);
      }
      if (TRAIN) {
        bool pr[R];
#pragma unroll
        for (int j = 0; j < R; ++j) pr[j] = valid[j] && (v[j] == nmin);
        const int nidx = last_label<R>(pr, L - 1);
        // every lane stores the same byte to the same address
        __builtin_amdgcn_raw_buffer_store_b8((unsigned char)nidx, dInorm, (live && store_ok) ? (int)sp : kDeadOffset, 0, 0);
      }
      st_p += ch.pstep;
  };
  // Trips of 2 D steps that lie inside the chain, on a chain without negative edge weights (the
  // band and the label scans hold for every step then): nothing in them asks whether a step is past
  // the end or which way its weight points, and the step for negative weights is not part of their
  // code.  A chain with such a weight takes the loop below from its first step.  Without argmin
  // labels, or with one label per lane (the scans of the usual training sizes with more labels
  // share their SIMDs and wait for memory, not for issue slots; their code is large enough as it is).
  int t0 = 1;
  if constexpr (!TRAIN || R == 1) {
    bool plain = true;
    if constexpr (KT >= 0 || KT == -2) {
      if (n > 2 * D) {  // (there is such a trip)
        bool bad = false;
        for (int i = lane; i < n; i += kWave) {
          const unsigned pi = (unsigned)(ch.pix0 + i * ch.pstep);
          const float wi = __builtin_bit_cast(
              float, __builtin_amdgcn_raw_buffer_load_b32(dW, (int)(pi * 4u), 0, 0));
          bad |= !(wi >= 0.f);
        }
        plain = ballot(bad) == 0;
      }
    }
    for (; plain && t0 + 2 * D <= n; t0 += 2 * D) {
#pragma unroll
      for (int u = 0; u < D; ++u) {
        // the loads of this ring slot were followed by at most D-1 steps' worth of memory operations
        wait_vmem<(D - 1) * kOps>();
        const PixF<R> px = ring[u];
        ring2[u] = load_next();
        step(px, t0 + u, std::true_type());
        // (the steps have no branch left between them; kept apart, the scalars of one step do not
        // pile up on those of the next, and none of them is spilled inside the loop)
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int u = 0; u < D; ++u) {
        wait_vmem<(D - 1) * kOps>();
        const PixF<R> px = ring2[u];
        ring[u] = load_next();
        step(px, t0 + D + u, std::true_type());
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  for (; t0 < n; t0 += 2 * D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      wait_vmem<(D - 1) * kOps>();
      const PixF<R> px = ring[u];
      ring2[u] = load_next();
      step(px, t0 + u, std::false_type());
    }
    if (t0 + D >= n) break;  // wave-uniform
#pragma unroll
    for (int u = 0; u < D; ++u) {
      wait_vmem<(D - 1) * kOps>();
      const PixF<R> px = ring2[u];
      ring[u] = load_next();
      step(px, t0 + D + u, std::false_type());
    }
  }
}

template <int R, bool VEC, bool MASK, bool TRAIN, int JACOBI>
__global__ void __launch_bounds__(kWave) sweep_fwd_kernel(const SweepParams p) {
  extern __shared__ __align__(16) float smem[];
  float* a_s = smem;            // kMaxL floats
  float* ctx_s = smem + kMaxL;  // L or L*L floats; several labels per lane: + the table moved down by one
  const int lane = threadIdx.x;
  const int L = p.L;
  const ChainCtx ch = locate_chain(p);
  if (!JACOBI && !p.pair_q && ch.n < 2) return;  // nothing to write

  CtxDesc desc;
  if (p.desc != nullptr) {
    desc = *p.desc;
  } else {
    desc.band_k = 0;
    desc.c0_is_min = 0;
    desc.cmax = 0.f;
    desc.msg_nonzero = 1;
    desc.linear = 0;
    desc.slope = 0.f;
  }
  // context table into LDS (dense path, run-time band taps, negative-weight fallback)
  if (R == 1 && desc.band_k == 0) {
    // full symmetric table for dense_step_r1: tab[fd * L + cd] = ctx(cd, fd), TRWP_forward.cu:101-113
    for (int i = lane; i < L * L; i += kWave) {
      const int fd = i / L, cd = i - fd * L;
      const int lo = cd < fd ? cd : fd, hi = cd < fd ? fd : cd;
      ctx_s[i] = p.ctx[p.ctx2d ? lo * L + hi : hi - lo];
    }
  } else {
    const int n_ctx = p.ctx2d ? L * L : L;
    for (int i = lane; i < n_ctx; i += kWave) ctx_s[i] = p.ctx[i];
    if (R > 1 && desc.band_k == 0) {  // (the dense scan is this kernel's step)
      float* c1_s = ctx_s + dense_c1_offset(L);
      for (int i = lane; i < dense_c1_floats(L); i += kWave) c1_s[i] = i + 1 < L ? p.ctx[i + 1] : 0.f;
      if (TRAIN) fill_dense_sym<R>(c1_s + dense_c1_floats(L), p.ctx, L, lane, kWave);
    }
  }
  __syncthreads();

  // Gauss-Seidel, chain-starved launches: the sweep of the opposite direction visits the same
  // pixels in reverse and depends on nothing but this chain's own first sweep, so the wavefront
  // runs it right away (p.fused_pair) instead of a second launch doing so.  What the first sweep
  // stored is read back by the same wavefront, in program order.
  const int halves = (!JACOBI && p.fused_pair) ? 2 : 1;
#pragma clang loop unroll(disable)
  for (int half = 0; half < halves; ++half) {
    ChainCtx c = ch;
    bool skip_s = p.skip_s_store != 0;
    if (half) {
      c.dir = ch.dir ^ 1;
      c.pix0 = ch.pix0 + (ch.n - 1) * ch.pstep;
      c.pstep = -ch.pstep;
      skip_s = p.skip_s_store2 != 0;
      wait_vmem<0>();
      __syncthreads();
    }
    // wide truncated-linear contexts: two label scans instead of 2K-1 taps or the dense scan
    if (desc.linear && !p.ctx2d && (desc.band_k == 0 || desc.band_k > 4)) {
      run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, -2>(p, desc, c, a_s, ctx_s, skip_s);
      continue;
    }
    // (a band whose entry 0 is not its smallest -- no Potts, linear or quadratic table -- takes the
    // taps at run time and reduces for the normalisation minimum)
    if (desc.band_k > 0 && !desc.c0_is_min) {
      run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, 0, false>(p, desc, c, a_s, ctx_s, skip_s);
      continue;
    }
    switch (desc.band_k) {
      case 0:
        if (R == 1 && L == 21)
          run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, (R == 1 ? -21 : -1)>(p, desc, c, a_s, ctx_s, skip_s);
        else
          run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, -1>(p, desc, c, a_s, ctx_s, skip_s);
        break;
      case 2: run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, 2, true>(p, desc, c, a_s, ctx_s, skip_s); break;
      case 3: run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, 3, true>(p, desc, c, a_s, ctx_s, skip_s); break;
      case 4: run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, 4, true>(p, desc, c, a_s, ctx_s, skip_s); break;
      default:
        // wider bands with the taps in registers: the table is constant from band_k on, so the
        // taps between band_k and the compiled width are the dense scan's own candidates
        // (only with several labels per lane: the short chains of small label counts gain nothing
        // and pay for the larger kernel)
        if constexpr (R >= 2) {
          if (desc.band_k <= 8) {
            run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, 8, true>(p, desc, c, a_s, ctx_s, skip_s);
            break;
          }
          if (desc.band_k <= 16) {
            run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, 16, true>(p, desc, c, a_s, ctx_s, skip_s);
            break;
          }
        }
        run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, 0, true>(p, desc, c, a_s, ctx_s, skip_s);
        break;
    }
  }
}

// A dense 1-D table in a launch with far fewer chains than the chip has SIMDs (p.split wavefronts
// per chain, chosen by the host; several labels per lane only).  Every wavefront of the workgroup
// runs the chain; see split_combine.
constexpr int kSplitMaxWaves = 8;
template <int R, bool VEC, bool MASK, bool TRAIN, int JACOBI>
__global__ void __launch_bounds__(kSplitMaxWaves * kWave) sweep_fwd_split_kernel(const SweepParams p) {
  extern __shared__ __align__(16) float smem[];
  const int L = p.L;
  float* a_s = smem;  // kMaxL floats per wavefront
  float* ctx_s = smem + (blockDim.x / kWave) * kMaxL;  // L floats, and the table moved down by one
  float* c1_s = ctx_s + dense_c1_offset(L);
  float* csym_s = c1_s + dense_c1_floats(L);
  float* xchg = csym_s + dense_sym_floats(R);
  const ChainCtx ch = locate_chain(p);
  if (!JACOBI && !p.pair_q && ch.n < 2) return;  // nothing to write (the same for every wavefront)
  CtxDesc desc;
  desc.band_k = 0;  // the dense scan is exact for any table; the descriptor only says whether
  desc.c0_is_min = 0;  // the initial messages are zero
  desc.cmax = 0.f;
  desc.msg_nonzero = p.desc != nullptr ? p.desc->msg_nonzero : 1;
  desc.linear = 0;
  desc.slope = 0.f;
  for (int i = threadIdx.x; i < L; i += blockDim.x) ctx_s[i] = p.ctx[i];
  for (int i = threadIdx.x; i < dense_c1_floats(L); i += blockDim.x) c1_s[i] = i + 1 < L ? p.ctx[i + 1] : 0.f;
  if (TRAIN) fill_dense_sym<R>(csym_s, p.ctx, L, (int)threadIdx.x, (int)blockDim.x);
  __syncthreads();
  const int halves = (!JACOBI && p.fused_pair) ? 2 : 1;
#pragma clang loop unroll(disable)
  for (int half = 0; half < halves; ++half) {
    ChainCtx c = ch;
    bool skip_s = p.skip_s_store != 0;
    if (half) {
      c.dir = ch.dir ^ 1;
      c.pix0 = ch.pix0 + (ch.n - 1) * ch.pstep;
      c.pstep = -ch.pstep;
      skip_s = p.skip_s_store2 != 0;
      wait_vmem<0>();
      __syncthreads();
    }
    run_chain_fwd<R, VEC, MASK, TRAIN, JACOBI, -3>(p, desc, c, a_s, ctx_s, skip_s, xchg);
  }
}

inline size_t split_lds_bytes(int L, int R, int waves, bool train) {
  return sizeof(float) * ((size_t)waves * kMaxL + dense_c1_offset(L) + dense_c1_floats(L) +
                          dense_sym_floats(R) + (size_t)2 * waves * kWave * (train ? 2 * R : R));
}

template <int R, bool VEC, bool MASK, bool TRAIN>
void launch_vm_split(const SweepParams& p, bool jacobi, hipStream_t st) {
  const int blocks = p.block_prefix[p.n_dirs];
  const int threads = p.split * kWave;
  const size_t lds = split_lds_bytes(p.L, R, p.split, TRAIN);
  const int mode = jacobi ? (p.u_fused ? 2 : 1) : 0;
  if (mode == 2)
    sweep_fwd_split_kernel<R, VEC, MASK, TRAIN, 2><<<blocks, threads, lds, st>>>(p);
  else if (mode == 1)
    sweep_fwd_split_kernel<R, VEC, MASK, TRAIN, 1><<<blocks, threads, lds, st>>>(p);
  else
    sweep_fwd_split_kernel<R, VEC, MASK, TRAIN, 0><<<blocks, threads, lds, st>>>(p);
}

template <int R, bool VEC, bool MASK, bool TRAIN>
void launch_vm(const SweepParams& p, bool jacobi, hipStream_t st) {
  if constexpr (R > 1) {
    if (p.split >= 2 && !p.ctx2d) {
      launch_vm_split<R, VEC, MASK, TRAIN>(p, jacobi, st);
      return;
    }
  }
  const int blocks = p.block_prefix[p.n_dirs];
  const size_t lds = fwd_lds_bytes(p.L, p.ctx2d);
  const int mode = jacobi ? (p.u_fused ? 2 : 1) : 0;
  if (mode == 2)
    sweep_fwd_kernel<R, VEC, MASK, TRAIN, 2><<<blocks, kWave, lds, st>>>(p);
  else if (mode == 1)
    sweep_fwd_kernel<R, VEC, MASK, TRAIN, 1><<<blocks, kWave, lds, st>>>(p);
  else
    sweep_fwd_kernel<R, VEC, MASK, TRAIN, 0><<<blocks, kWave, lds, st>>>(p);
}

}  // namespace

// (the scans that keep argmin labels and those that do not are compiled as separate units)
template <int R, bool TRAIN>
void launch_sweep_fwd_t(const SweepParams& p, bool jacobi, hipStream_t st) {
  if (p.block_prefix[p.n_dirs] <= 0) return;
  const bool mask = p.L != R * kWave;
  // one descriptor per plane for the whole kernel: whole lanes of labels, and, where some lanes have
  // none, an image of at most 2 GiB (run_chain_fwd, foff_ok)
  const bool vec = (p.L % R) == 0 &&
                   (!mask || (int64_t)p.H * p.W * p.L * 4 <= (int64_t)1 << 31);
  if constexpr (R > 1) {
    if (!vec) {
      launch_vm<R, false, true, TRAIN>(p, jacobi, st);
      return;
    }
  }
  if (mask)
    launch_vm<R, true, true, TRAIN>(p, jacobi, st);
  else
    launch_vm<R, true, false, TRAIN>(p, jacobi, st);
}

template void launch_sweep_fwd_t<MPL_INST_R, (MPL_INST_TRAIN != 0)>(const SweepParams&, bool, hipStream_t);

}  // namespace mpl
