// Shared device helpers of the TRWP / ISGMR kernels for gfx950 (CDNA4, wave64).
//
// Mapping used by every scan kernel: one 64-lane wavefront walks one chain (a row, column or
// diagonal segment) of one direction.  The L labels of a pixel are spread over the lanes in
// blocks: lane i owns labels R*i .. R*i+R-1 with R = ceil(L/64).  A pixel's label vector is then
// one R-dword buffer access per lane, a one-label shift is a single DPP wave shift plus register
// renaming, and the min / sum over labels is a DPP reduction.
//
// Memory is accessed through buffer descriptors whose base is the first label vector of the batch
// item.  The offset of an access is (pixel offset `so`) + (offset of the lane's labels); it is
// range-checked against num_records, so every access passes num_records = so + (size of one label
// vector): lanes whose labels do not exist fall outside the descriptor, their loads return 0 and
// their stores are dropped by the hardware.  The whole offset travels in the vector-offset operand
// (none in the scalar-offset register): multi-dword stores that used a scalar-offset register had
// their data overwritten by the instructions that followed them on the MI355X.  This keeps the
// scan loop free of branches around memory instructions, which is what lets the loads of the next
// pixels stay in flight (the hardware counter the compiler waits on counts memory operations in
// order, so a branch that may skip one forces a conservative wait).  Offsets are 32-bit: one image
// (H*W*L floats) must stay below 4 GiB; batch items are reached through the base.
#ifndef MPLAYERS_AMD_MP_COMMON_H_
#define MPLAYERS_AMD_MP_COMMON_H_

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "../../include/mplayers_amd.h"

namespace mpl {

constexpr int kWave = 64;
constexpr int kMaxL = MPL_MAX_LABELS;
constexpr int kMaxDirs = MPL_MAX_DIRS;
constexpr int kMaxCtx2dL = 64;  // (L,L) context table kept in LDS
constexpr int kMaxBandK = 32;   // widest band handled by the O(L*K) path

#ifndef MPL_PREFETCH
#define MPL_PREFETCH 8
#endif
constexpr int kPrefetch = MPL_PREFETCH;  // upper limit of pixels in flight per wave

// The hardware counter of outstanding vector-memory operations of a wave has 6 bits (63 at most).
// The prefetch ring is sized from the number of memory instructions a step issues so that a wave
// never has more than kMaxInFlight of them outstanding: the explicit waits of the scan loops then
// stay exact, and a deeper ring buys nothing (2 to 8 pixels ahead measure the same).
#ifndef MPL_MAX_INFLIGHT
#define MPL_MAX_INFLIGHT 52
#endif
constexpr int kMaxInFlight = MPL_MAX_INFLIGHT;
constexpr int ring_depth(int ops_per_step) {
  int d = kMaxInFlight / (ops_per_step > 0 ? ops_per_step : 1);
  return d < 1 ? 1 : (d > kPrefetch ? kPrefetch : d);
}
// Explicit wait until at most N vector-memory operations of this wave are outstanding (gfx9
// encoding of s_waitcnt: vmcnt in bits [3:0] and [15:14]; the other counters left at their maxima).
template <int N>
__device__ __forceinline__ void wait_vmem() {
  constexpr int n = N > 62 ? 62 : (N < 0 ? 0 : N);
  __builtin_amdgcn_s_waitcnt((n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

// Scheduling fence between the groups of loads that fill the prefetch ring before a scan loop.
#define MPL_ORDER_LOADS() __builtin_amdgcn_sched_barrier(0)

// number of instructions one R-label access of floats / of bytes takes
constexpr int vec_ops(int R, bool vec) { return vec ? 1 : R; }
constexpr int byte_ops(int R, bool vec) { return (vec && (R == 4 || R == 2)) ? 1 : R; }

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
// the same shifts where the lane without a source keeps its own value of x: in place, with no fill
// register to set up.  For a vector that an earlier filling shift in the same direction produced,
// that lane already holds the fill, and keeps holding it.
__device__ __forceinline__ float wave_shl1_keep(float x) { return dpp_f<0x130>(x, x); }
__device__ __forceinline__ float wave_shr1_keep(float x) { return dpp_f<0x138>(x, x); }

__device__ __forceinline__ float readlane_f(float x, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}
// tells the compiler that x is wave-uniform (keeps addressing in scalar registers)
__device__ __forceinline__ int uniform_i(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ float uniform_f(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
}

// Order-preserving map between the bits of a float and a signed integer (its own inverse):
// x < y  <=>  float_key(x) < float_key(y), with -0 below +0.
__device__ __forceinline__ int float_key(int bits) { return bits ^ ((bits >> 31) & 0x7fffffff); }

// min over the 64 lanes, returned wave-uniform.  The reduction runs on the integer keys: an integer
// minimum folds each lane shift into the min instruction itself (the shifted-in lanes read the
// identity INT_MAX), which the compiler does not do for a float minimum.
__device__ __forceinline__ float wave_min(float x) {
  const int top = 0x7fffffff;
  int k = float_key(__builtin_bit_cast(int, x));
  auto imin = [](int a, int b) { return a < b ? a : b; };
  k = imin(k, __builtin_amdgcn_update_dpp(top, k, 0x111, 0xf, 0xf, false));  // row_shr:1
  k = imin(k, __builtin_amdgcn_update_dpp(top, k, 0x112, 0xf, 0xf, false));  // row_shr:2
  k = imin(k, __builtin_amdgcn_update_dpp(top, k, 0x114, 0xf, 0xf, false));  // row_shr:4
  k = imin(k, __builtin_amdgcn_update_dpp(top, k, 0x118, 0xf, 0xf, false));  // row_shr:8: lane 15 of each row holds the row min
  k = imin(k, __builtin_amdgcn_update_dpp(top, k, 0x142, 0xa, 0xf, false));  // row_bcast:15 into rows 1 and 3
  k = imin(k, __builtin_amdgcn_update_dpp(top, k, 0x143, 0xc, 0xf, false));  // row_bcast:31 into rows 2 and 3
  return __builtin_bit_cast(float, float_key(__builtin_amdgcn_readlane(k, 63)));
}

// the same on the float values themselves (three instructions per step instead of one, but no
// conversions before and after: the shorter path where little else overlaps the reduction)
__device__ __forceinline__ float wave_min_f32(float x) {
  const float inf = INFINITY;
  x = fminf(x, dpp_f<0x111>(inf, x));
  x = fminf(x, dpp_f<0x112>(inf, x));
  x = fminf(x, dpp_f<0x114>(inf, x));
  x = fminf(x, dpp_f<0x118>(inf, x));
  x = fminf(x, dpp_f<0x142, 0xa>(inf, x));
  x = fminf(x, dpp_f<0x143, 0xc>(inf, x));
  return readlane_f(x, 63);
}

// The float minimum with each lane shift folded into the min instruction, which the compiler does
// not emit by itself: v_min_f32 with a DPP source, in place, so that a lane without a source keeps
// its own value.  No conversions to integer keys and back: 6 instructions and the read-out.  (A
// DPP operand written by the instruction before needs two wait states, which the compiler cannot
// see inside the statement: each instruction carries its own, in one statement, since the
// compiler pads the gap between two statements itself.)
__device__ __forceinline__ float wave_min_fast(float x) {
#define MPL_MIN_DPP(CTRL) "s_nop 1\n\tv_min_f32_dpp %0, %0, %0 " CTRL " bank_mask:0xf\n\t"
  asm(MPL_MIN_DPP("row_shr:1 row_mask:0xf") MPL_MIN_DPP("row_shr:2 row_mask:0xf")
      MPL_MIN_DPP("row_shr:4 row_mask:0xf") MPL_MIN_DPP("row_shr:8 row_mask:0xf")
      MPL_MIN_DPP("row_bcast:15 row_mask:0xa") MPL_MIN_DPP("row_bcast:31 row_mask:0xc") "s_nop 0"
      : "+v"(x));
#undef MPL_MIN_DPP
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

// The same with each lane shift folded into the add, like wave_min_fast (a lane without a source
// keeps its value, which is what adding zero gives): 6 instructions instead of 10, but one block
// that the compiler cannot spread other work into.  For steps of a wavefront that has its SIMD to
// itself, where every issue slot counts; where several wavefronts share a SIMD the version above,
// whose gaps the compiler fills, is the faster one.  Both give the same bits.
__device__ __forceinline__ float wave_sum_fast(float x) {
#define MPL_ADD_DPP(CTRL) "s_nop 1\n\tv_add_f32_dpp %0, %0, %0 " CTRL " bank_mask:0xf\n\t"
  asm(MPL_ADD_DPP("row_shr:1 row_mask:0xf") MPL_ADD_DPP("row_shr:2 row_mask:0xf")
      MPL_ADD_DPP("row_shr:4 row_mask:0xf") MPL_ADD_DPP("row_shr:8 row_mask:0xf")
      MPL_ADD_DPP("row_bcast:15 row_mask:0xa") MPL_ADD_DPP("row_bcast:31 row_mask:0xc") "s_nop 0"
      : "+v"(x));
#undef MPL_ADD_DPP
  return readlane_f(x, 63);
}

__device__ __forceinline__ uint64_t ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }

template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf>
__device__ __forceinline__ int dpp_i(int old, int src) {
  return __builtin_amdgcn_update_dpp(old, src, CTRL, ROW_MASK, BANK_MASK, false);
}

// Inclusive scans over the 64 lanes.  Prefix: lane i gets the result over lanes 0..i (shifts within
// the rows of 16 lanes, then the row totals travel through the row broadcasts).  Suffix: lane i
// gets the result over lanes i..63 (there is no broadcast in that direction: the three later row
// totals are read back as scalars).
// (the float scans run on the order-preserving integer keys, as wave_min does)
__device__ __forceinline__ float lane_prefix_min(float x) {
  constexpr int hi = 0x7fffffff;
  int k = float_key(__builtin_bit_cast(int, x));
  k = min(k, dpp_i<0x111>(hi, k));
  k = min(k, dpp_i<0x112>(hi, k));
  k = min(k, dpp_i<0x114>(hi, k));
  k = min(k, dpp_i<0x118>(hi, k));
  k = min(k, dpp_i<0x142, 0xa>(hi, k));
  k = min(k, dpp_i<0x143, 0xc>(hi, k));
  return __builtin_bit_cast(float, float_key(k));
}
__device__ __forceinline__ int lane_prefix_max(int x) {
  constexpr int lo = -0x7fffffff - 1;
  x = max(x, dpp_i<0x111>(lo, x));
  x = max(x, dpp_i<0x112>(lo, x));
  x = max(x, dpp_i<0x114>(lo, x));
  x = max(x, dpp_i<0x118>(lo, x));
  x = max(x, dpp_i<0x142, 0xa>(lo, x));
  x = max(x, dpp_i<0x143, 0xc>(lo, x));
  return x;
}
__device__ __forceinline__ int lane_suffix_min(int x, int lane) {
  constexpr int hi = 0x7fffffff;
  x = min(x, dpp_i<0x101>(hi, x));
  x = min(x, dpp_i<0x102>(hi, x));
  x = min(x, dpp_i<0x104>(hi, x));
  x = min(x, dpp_i<0x108>(hi, x));
  const int r1 = __builtin_amdgcn_readlane(x, 16), r2 = __builtin_amdgcn_readlane(x, 32),
            r3 = __builtin_amdgcn_readlane(x, 48);
  const int m2 = min(r2, r3), m1 = min(r1, m2);
  const int row = lane >> 4;
  const int later = row == 0 ? m1 : (row == 1 ? m2 : (row == 2 ? r3 : hi));
  return min(x, later);
}

__device__ __forceinline__ float lane_suffix_min(float x, int lane) {
  return __builtin_bit_cast(float, float_key(lane_suffix_min(float_key(__builtin_bit_cast(int, x)), lane)));
}

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
// buffer access.  A descriptor covers `bytes` bytes at p; accesses beyond it read 0 / are dropped.
// ------------------------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x3 __attribute__((ext_vector_type(3)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x3 __attribute__((ext_vector_type(3)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ rsrc_t make_rsrc(const void* p, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// Cache-policy bits of the label-vector accesses (gfx94x/95x: 1 = sc0, 2 = nt, 16 = sc1).  Every
// plane is streamed once per sweep and is far larger than the caches, so loads and stores carry the
// non-temporal hint; measured on the 1500x2000x192 forward sweep: 2.98 ms without, 2.54 ms with
// (with the present kernels 2.15 ms against 2.39 ms with the hint on the loads only, 2.17 ms on the
// stores only, and 3.48 ms with sc1 added to both).
#ifndef MPL_LD_AUX
#define MPL_LD_AUX 2
#endif
#ifndef MPL_ST_AUX
#define MPL_ST_AUX 2
#endif

constexpr int kDeadOffset = 0x7ffffff0;  // a vector offset no descriptor covers: access suppressed
// the same for descriptors that cover a whole image (up to kMaxImageBytes, beyond 2 GiB)
constexpr unsigned kDeadWide = 0xfffffff0u;
constexpr int64_t kMaxImageBytes = 0xffffffc0ll;

// R consecutive floats at vector byte offset `off` (range-checked) + scalar byte offset `so`.
// VEC: one R-dword access (used when every lane's block lies entirely inside or entirely outside
// the pixel vector, i.e. L % R == 0); otherwise R single-dword accesses, each checked on its own.
template <int R, bool VEC>
__device__ __forceinline__ void buf_load(rsrc_t r, int off, unsigned so, float (&x)[R]) {
  if constexpr (VEC && R == 2) {
    f32x2 t = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(r, (int)((unsigned)off + so), 0, MPL_LD_AUX));
    x[0] = t[0];
    x[1] = t[1];
  } else if constexpr (VEC && R == 3) {
    f32x3 t = __builtin_bit_cast(f32x3, __builtin_amdgcn_raw_buffer_load_b96(r, (int)((unsigned)off + so), 0, MPL_LD_AUX));
    x[0] = t[0];
    x[1] = t[1];
    x[2] = t[2];
  } else if constexpr (VEC && R == 4) {
    f32x4 t = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)((unsigned)off + so), 0, MPL_LD_AUX));
    x[0] = t[0];
    x[1] = t[1];
    x[2] = t[2];
    x[3] = t[3];
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j)
      x[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)((unsigned)(off + 4 * j) + so), 0, MPL_LD_AUX));
  }
}

template <int R, bool VEC>
__device__ __forceinline__ void buf_store(rsrc_t r, int off, unsigned so, const float (&x)[R]) {
  if constexpr (VEC && R == 2) {
    f32x2 t = {x[0], x[1]};
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, t), r, (int)((unsigned)off + so), 0, MPL_ST_AUX);
  } else if constexpr (VEC && R == 3) {
    f32x3 t = {x[0], x[1], x[2]};
    __builtin_amdgcn_raw_buffer_store_b96(__builtin_bit_cast(u32x3, t), r, (int)((unsigned)off + so), 0, MPL_ST_AUX);
  } else if constexpr (VEC && R == 4) {
    f32x4 t = {x[0], x[1], x[2], x[3]};
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, t), r, (int)((unsigned)off + so), 0, MPL_ST_AUX);
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j)
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[j]), r, (int)((unsigned)(off + 4 * j) + so), 0, MPL_ST_AUX);
  }
}

// R consecutive uint8 at byte offset `off`
template <int R, bool VEC>
__device__ __forceinline__ void buf_load_u8(rsrc_t r, int off, unsigned so, int (&x)[R]) {
  if constexpr (VEC && R == 4) {
    unsigned t = __builtin_amdgcn_raw_buffer_load_b32(r, (int)((unsigned)off + so), 0, MPL_LD_AUX);
    x[0] = t & 0xff;
    x[1] = (t >> 8) & 0xff;
    x[2] = (t >> 16) & 0xff;
    x[3] = t >> 24;
  } else if constexpr (VEC && R == 2) {
    unsigned t = __builtin_amdgcn_raw_buffer_load_b16(r, (int)((unsigned)off + so), 0, MPL_LD_AUX);
    x[0] = t & 0xff;
    x[1] = (t >> 8) & 0xff;
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j) x[j] = __builtin_amdgcn_raw_buffer_load_b8(r, (int)((unsigned)(off + j) + so), 0, MPL_LD_AUX);
  }
}

template <int R, bool VEC>
__device__ __forceinline__ void buf_store_u8(rsrc_t r, int off, unsigned so, const int (&x)[R]) {
  if constexpr (VEC && R == 4) {
    unsigned t = (unsigned)x[0] | ((unsigned)x[1] << 8) | ((unsigned)x[2] << 16) | ((unsigned)x[3] << 24);
    __builtin_amdgcn_raw_buffer_store_b32(t, r, (int)((unsigned)off + so), 0, MPL_ST_AUX);
  } else if constexpr (VEC && R == 2) {
    unsigned short t = (unsigned short)((unsigned)x[0] | ((unsigned)x[1] << 8));
    __builtin_amdgcn_raw_buffer_store_b16(t, r, (int)((unsigned)off + so), 0, MPL_ST_AUX);
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j)
      __builtin_amdgcn_raw_buffer_store_b8((unsigned char)x[j], r, (int)((unsigned)(off + j) + so), 0, MPL_ST_AUX);
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
    // enumerate so that chain lengths first grow, then (second branch) shrink, whatever the sign of
    // the column step: with the lengths of a diagonal sweep ordered long-first the SIMDs that drew
    // several long chains finished 15 % later than the rest
    if (g.ws > 0) ww = W - 1 - ww;
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

struct ChainCtx {
  int bv;     // batch item
  int pix0;   // pixel index of the chain start inside its image
  int pstep;  // pixel stride along the chain
  int n;      // pixels in the chain
  int dir;
};

// which (direction, batch item, chain) a workgroup owns
template <typename Params>
__device__ __forceinline__ ChainCtx locate_chain(const Params& p) {
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
  ch.bv = bv;
  ch.pix0 = h0 * p.W + w0;
  ch.pstep = g.hs * p.W + g.ws;
  ch.n = n;
  ch.dir = dir;
  return ch;
}

// ------------------------------------------------------------------------------------------------
// context descriptor, computed on the device so that no host round trip is needed
// ------------------------------------------------------------------------------------------------
struct CtxDesc {
  int band_k;     // > 0: c[k] == cmax for all k >= band_k and c[k] <= cmax below; 0: dense path
  int c0_is_min;  // c[0] <= c[k] for all k
  float cmax;
  int msg_nonzero;  // set by the belief pass when some initial message is not zero
  int linear;       // c[k] == min(slope * k, c[L-1]) exactly for every k, slope >= 0 (truncated linear)
  float slope;
};

// ------------------------------------------------------------------------------------------------
// kernel parameter blocks
// ------------------------------------------------------------------------------------------------
struct SweepParams {
  int B, H, W, L;
  int ctx2d;
  int n_dirs;                      // directions in this launch
  int dirs[kMaxDirs];              // their ids
  int block_prefix[kMaxDirs + 1];  // prefix sums of B * n_chains
  float rho;
  const float* belief;             // S plane (N)
  float* belief_out;               // TRWP: == belief; Jacobi: unused
  const float* msg_in;             // (n_dir_total, N) planes read
  float* msg_out;                  // (n_dir_total, N) planes written
  const float* edge;               // (n_dir_total, P)
  const float* ctx;
  const CtxDesc* desc;             // may be null: dense path
  uint8_t* idx_min;                // (n_dir_total, N) of this iteration, or null
  uint8_t* idx_norm;               // (n_dir_total, P) of this iteration, or null
  int pack;                        // packed scans (mp_pack.hip): chains per wavefront; 0: one chain per
                                   // wavefront.  Decided once per launch by the host (mp_api.hip)
  int split;                       // dense 1-D table, several labels per lane, few chains: wavefronts
                                   // per chain that share the front labels of a pixel (0, 1: one)
  int pair_q;                      // Gauss-Seidel: belief plane holds Q between the sweeps of a pair
  int skip_s_store;                // Gauss-Seidel: last sweep of the call, nobody reads S after it
  int fused_pair;                  // Gauss-Seidel: every wavefront sweeps dirs[0], then dirs[0] ^ 1
  int skip_s_store2;               // skip_s_store of that second sweep
  int first_iter;                  // Gauss-Seidel: first iteration (planes not yet swept hold the
                                   // caller's initial messages, which need not be read when zero)
  int u_pair_share;                // Jacobi: directions d and d^1 read the U plane of the even one
  int64_t u_stride;                // Jacobi: elements between the U planes of msg_in (0: all directions
                                   // read the one plane at msg_in)
  int u_fused;                     // Jacobi, four directions, rho == 1: `belief` is the unary and msg_in
                                   // holds the old messages themselves; the scans form U on the fly
  int zero_start;                  // Gauss-Seidel: store zeros at the chain start of msg_out (the
                                   // caller's buffer is undefined and this is its first sweep)
  int zero_first;                  // first sweeps over messages the device found to be all zero
                                   // (CtxDesc::msg_nonzero == 0): `belief_zero` stands for the plane the
                                   // sweep would read (Gauss-Seidel, first pair of directions: the belief
                                   // plane, which then need not exist; Jacobi, first iteration: U), and
                                   // the even sweep of that pair stores no plane
  const float* belief_zero;        // the unary terms
  float* edge_label;               // soft TRWP: (n_dir_total, P, L, L) duals of this iteration, or null
};

struct BackParams {
  int B, H, W, L;
  int ctx2d;
  int n_dirs;
  int dirs[kMaxDirs];
  int block_prefix[kMaxDirs + 1];
  float rho;
  // TRWP: g_k = A + h_k.  a_in: plane read as A (dcost_final on the first sweep), a_out: dunary.
  const float* a_in;
  float* a_out;
  float* h;                 // (n_dir_total, N) planes h_k
  int first_touch;          // h_dir and h_inv have not been written yet: read as zero
  int inv_from_a;           // h_inv == -A (the previous launch swept the opposite direction)
  int skip_hd_store;        // h_dir is not read again before it is overwritten (or ever)
  int skip_hi_store;        // h_inv is never read again (last sweeps of the backward pass)
  int fused_pair;           // Gauss-Seidel: every wavefront walks dirs[0] (odd), then dirs[0] ^ 1
  int skip_h2;              // that second walk stores neither h plane (last iteration walked)
  // ISGMR: gu_in planes (plane stride gu_stride; 0 on the first iteration where gu_k = dcost_final),
  // du_out (n_dir_total, N) receives dU_d in place of gu_d
  const float* gu_in;
  int64_t gu_stride;
  int gu_pair_share;        // directions d and d^1 read the gu plane of the even one
  float* du_out;
  const float* edge;        // (n_dir_total, P)
  const float* ctx;
  const uint8_t* idx_min;   // (n_dir_total, N) of this iteration
  const uint8_t* idx_norm;  // (n_dir_total, P)
  float* dedge;             // (n_dir_total, P) accumulates; null: not wanted, that part of the step is left out
  float* dctx;              // accumulates; null: not wanted
  int same_label;           // dctx also collects the pairs with cd == fd (the hard operator of the
                            // reference's TRWP_hard_soft build, TRWP_hard_soft/TRWP_backward.cu:104-111)
  const float* edge_label;  // soft TRWP: (n_dir_total, P, L, L) duals of this iteration
  int pack;                 // packed scans (mp_pack.hip): chains per wavefront
};

// records the message mpl_last_error() returns on this thread and returns `code`
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// MPL_OPT_CPU_THREADS (cpu/mp_cpu.cpp)
int set_cpu_threads(int n);

// launchers, one translation unit per R so that the instantiations compile in parallel
template <int R, bool TRAIN>
void launch_sweep_fwd_t(const SweepParams& p, bool jacobi, hipStream_t st);
template <int R>
inline void launch_sweep_fwd(const SweepParams& p, bool train, bool jacobi, hipStream_t st) {
  if (train)
    launch_sweep_fwd_t<R, true>(p, jacobi, st);
  else
    launch_sweep_fwd_t<R, false>(p, jacobi, st);
}
template <int R>
void launch_sweep_bwd(const BackParams& p, bool jacobi, hipStream_t st);

// Launch policy of the current device.  The scans put one wavefront on a chain, so which kernel a
// launch takes depends on how many wavefronts' worth of chains it has per SIMD (four SIMDs per
// compute unit): the thresholds are multiples of the device's SIMD count, read from its properties
// once per device.  The multiples were measured on an MI355X (256 compute units, 1024 SIMDs).
struct LaunchPolicy {
  int n_simd;
  // Gauss-Seidel launches of at most this many wavefronts (one per SIMD) run both sweeps of a pair
  // of opposite directions in one launch
  int fused_pair_max_waves;
  // A launch is packed (mp_pack.hip: several chains per wavefront, at most kPackedMaxL labels) by
  // default when
  //  * its table is 2-D (a learned table, dense) and it has more chains than SIMDs; with 21 labels,
  //    whose one-chain-per-wavefront scans have a short step of their own, more chains than two
  //    wavefronts per SIMD,
  //  * its table is 1-D and it has at most 8 labels and more than 6 chains per SIMD, or at most 16
  //    labels and more than 9.  The packed step is the dense one, L candidates per label, whatever
  //    the table; nearly every 1-D table is a band (Potts, truncated linear or quadratic), whose step
  //    in the one-chain scans takes a few taps, and only the device knows which it is: these are the
  //    sizes from which packing pays for a band, too.  A caller with dense 1-D tables of up to 32
  //    labels and thousands of chains per launch passes MPL_F_PACKED_ALWAYS.
  int packed_min_chains;       // 2-D table
  int packed_min_chains21;     // 2-D table, 21 labels
  int packed_min_chains_1d8;   // 1-D table, at most 8 labels
  int packed_min_chains_1d16;  // 1-D table, 9 to 16 labels
  // reverse scans with one label per lane: launches of at most this many chains (two wavefronts per
  // SIMD) are taken to be bound by the latency of a step (mp_bwd.hip)
  int direct_max_chains;
};
const LaunchPolicy& launch_policy();  // mp_api.hip

// packed scans for small label counts (mp_pack.hip): several chains per wavefront.
constexpr int kPackedMaxL = 32;
// chains per wavefront the packed scans would use for such a launch (below 2: they do not apply);
// always: pack whatever the table and the number of chains (tests, comparisons, such callers)
int packed_chains_per_wave(int B, int H, int W, int L, bool ctx2d, int64_t chains, bool always);
// G: what packed_chains_per_wave returned for the launch (>= 2)
void launch_packed_fwd(const SweepParams& p, bool train, bool jacobi, int G, hipStream_t st);
void launch_packed_bwd(const BackParams& p, bool jacobi, int G, hipStream_t st);

// soft-weighted TRWP (mp_soft.hip): one direction per launch, L <= 64
void launch_soft_fwd(const SweepParams& p, bool train, hipStream_t st);
void launch_soft_bwd(const BackParams& p, hipStream_t st);
void launch_swm_fwd(const float* msg, int n_trees, int L, float* out, uint8_t* min_ind,
                    hipStream_t st);
void launch_swm_bwd(const float* dout, const float* msg, const uint8_t* min_ind, int n_trees, int L,
                    float* dmsg, hipStream_t st);

// LDS of the forward scan with several labels per lane: after the 1-D table c[0 .. L-1] (padded to
// whole groups of four) stands the table moved down by one entry, c1[i] = c[i + 1], which the dense
// scan reads four entries at a time up to two trips past the last label
__host__ __device__ inline int dense_c1_offset(int L) { return (L + 3) & ~3; }
__host__ __device__ inline int dense_c1_floats(int L) { return ((L + 3) & ~3) + 32; }

// Front labels per wavefront where `waves` wavefronts scan a pixel together: whole trips of the
// dense scan (4 R front labels)
__host__ __device__ inline int split_share(int L, int R, int waves) {
  const int trip = 4 * R;
  return ((L + trip * waves - 1) / (trip * waves)) * trip;
}

// ... and, for the argmin labels of the dense scan, the table around its centre: entries for every
// difference of two labels that R * 64 lanes of labels can form
__host__ __device__ inline int dense_sym_floats(int R) { return 2 * R * kWave; }

inline size_t fwd_lds_bytes(int L, int ctx2d) {
  if (ctx2d || L <= kWave) return sizeof(float) * (kMaxL + L * L);
  const int R = (L + kWave - 1) / kWave;
  return sizeof(float) * (kMaxL + dense_c1_offset(L) + dense_c1_floats(L) + dense_sym_floats(R));
}

}  // namespace mpl

#endif  // MPLAYERS_AMD_MP_COMMON_H_
