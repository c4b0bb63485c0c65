// Bandwidth probes: what the memory system sustains for traffic of the scans' shape; and, at the end
// of the file, an issue probe: what instruction patterns cost a lone wavefront.
//
// The scan kernels are long-lived wavefronts, one per chain, that stream several planes in and out
// one pixel vector at a time.  These kernels move the same bytes in the same shape without any of
// the arithmetic (n_in planes read and summed, n_out planes written, register prefetch ring), and a
// one-pass streaming kernel moves them the way an element-wise kernel does, so the scans can be
// rated against what the hardware delivers for their access pattern rather than against the data
// sheet alone.  Diagnostics only; no counterpart in the reference.  Built into a library of its own
// (libmplayers_probe.so, mp_probe.h) that only the benchmark and the tests load.

#include <stdarg.h>
#include <stdio.h>

#include "mp_common.h"
#include "mp_probe.h"

using namespace mpl;

namespace {

constexpr int kEinval = -1, kElaunch = -2;
thread_local char g_probe_err[256] = "";
int pfail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int pfail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_probe_err, sizeof(g_probe_err), fmt, ap);
  va_end(ap);
  return code;
}

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kProbeDepth = 8;  // pixels in flight per wavefront, as in the scans

// One wavefront per chain; a pixel vector is `units` 16-byte pieces (lanes beyond that idle).
// Chain c starts at unit c * chain_stride, pixel t at + t * pix_stride.
template <int NIN, int NOUT>
__global__ void __launch_bounds__(kWave) chain_copy_kernel(const v4f* __restrict__ in,
                                                           v4f* __restrict__ out, int64_t plane,
                                                           int units, int64_t chain_stride,
                                                           int64_t pix_stride, int n_pix) {
  if ((int)threadIdx.x >= units) return;
  const int64_t base = (int64_t)blockIdx.x * chain_stride + threadIdx.x;
  v4f ring[kProbeDepth][NIN];
  v4f total = 0.f;
#pragma unroll
  for (int d = 0; d < kProbeDepth; ++d)
#pragma unroll
    for (int k = 0; k < NIN; ++k)
      ring[d][k] = __builtin_nontemporal_load(in + k * plane + base + (d < n_pix ? d : 0) * pix_stride);
  for (int t = 0; t < n_pix; t += kProbeDepth) {
#pragma unroll
    for (int d = 0; d < kProbeDepth; ++d) {
      v4f acc = ring[d][0];
#pragma unroll
      for (int k = 1; k < NIN; ++k) acc += ring[d][k];
      const int next = t + d + kProbeDepth;
      if (next < n_pix) {
#pragma unroll
        for (int k = 0; k < NIN; ++k)
          ring[d][k] = __builtin_nontemporal_load(in + k * plane + base + next * pix_stride);
      }
      if (t + d < n_pix) {
#pragma unroll
        for (int k = 0; k < NOUT; ++k)
          __builtin_nontemporal_store(acc + (float)k, out + k * plane + base + (t + d) * pix_stride);
        if (NOUT == 0) total += acc;
      }
    }
  }
  if (NOUT == 0 && total.x == 1.2345e30f) out[base] = total;  // keeps the loads alive
}

// One thread per 16 bytes, one pass, as the element-wise kernels.
template <int NIN, int NOUT>
__global__ void __launch_bounds__(256) stream_copy_kernel(const v4f* __restrict__ in,
                                                          v4f* __restrict__ out, int64_t plane) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= plane) return;
  v4f acc = __builtin_nontemporal_load(in + i);
#pragma unroll
  for (int k = 1; k < NIN; ++k) acc += __builtin_nontemporal_load(in + k * plane + i);
#pragma unroll
  for (int k = 0; k < NOUT; ++k) __builtin_nontemporal_store(acc + (float)k, out + k * plane + i);
  if (NOUT == 0 && acc.x == 1.2345e30f) out[i] = acc;
}

template <int NIN, int NOUT>
void launch_probe(int shape, const float* in, float* out, int H, int W, int L, hipStream_t st) {
  const int units = L / 4;
  const int64_t plane = (int64_t)H * W * units;
  const v4f* src = reinterpret_cast<const v4f*>(in);
  v4f* dst = reinterpret_cast<v4f*>(out);
  if (shape == MPLP_ROWS) {
    chain_copy_kernel<NIN, NOUT><<<H, kWave, 0, st>>>(src, dst, plane, units, (int64_t)W * units,
                                                      units, W);
  } else if (shape == MPLP_COLUMNS) {
    chain_copy_kernel<NIN, NOUT><<<W, kWave, 0, st>>>(src, dst, plane, units, units,
                                                      (int64_t)W * units, H);
  } else {
    stream_copy_kernel<NIN, NOUT><<<(unsigned)((plane + 255) / 256), 256, 0, st>>>(src, dst, plane);
  }
}


// ------------------------------------------------------------------------------------------------
// Issue probe: what instruction patterns cost a wavefront that has its SIMD to itself.  One
// wavefront runs a few hundred copies of each pattern between two reads of the shader clock; the
// difference, less that of an empty region, divided by the number of issue slots is reported.
// The scans of launches with fewer chains than the chip has SIMDs are bound by exactly these costs.
// ------------------------------------------------------------------------------------------------
struct IssuePattern {
  const char* name;
  int slots;  // instructions (idle slots included) between the two clock reads
};
const IssuePattern kIssuePatterns[] = {
    {"empty region", 0},
    {"vop2 add, independent", 480},
    {"vop2 add, each needs the one before", 480},
    {"vop2 multiply-add (v_fmac)", 480},
    {"vop3 multiply-add (v_fma), three registers", 480},
    {"vop3 multiply-add, two registers and a scalar", 480},
    {"v_min3, three registers", 480},
    {"comparison into a scalar mask", 480},
    {"select on a scalar mask, registers", 480},
    {"select on a scalar mask, inline constant", 480},
    {"comparison, two idle slots, select (3 slots)", 480},
    {"two comparisons and two selects interleaved (4 slots)", 480},
    {"s_nop 0", 480},
    {"s_nop 1", 480},
    {"scalar add", 480},
    {"v_readlane", 480},
    {"two idle slots and a lane-shift minimum (2 slots)", 480},
    {"lane-shift minimum and two independent adds (3 slots)", 480},
    {"v_exp", 480},
    {"v_rcp", 480},
    {"ds_bpermute x8, one wait (9 slots)", 477},
    {"ds_bpermute and wait (round trip, 2 slots)", 480},
    {"ds_read_b32 and wait (round trip, 2 slots)", 480},
    {"ds_add_f32, ds_wrxchg_rtn and wait, distinct addresses (3 slots)", 480},
    {"ds_add_f32 of 64 lanes to one address and wait (2 slots)", 480},
};
constexpr int kNumIssuePatterns = (int)(sizeof(kIssuePatterns) / sizeof(kIssuePatterns[0]));

// %0: byte address of this lane's LDS word, %1: that of word 0.  They are operands of every
// statement, so whatever the compiler does with its registers between two statements, an LDS
// access of a pattern never sees an address it did not get from the compiler.  v10..v17 and the
// scalar registers only feed arithmetic whose result is not read: what they hold does not matter.
#define MPL_ISSUE_TIMED(idx, body)                                                                \
  {                                                                                               \
    __builtin_amdgcn_s_barrier();                                                                 \
    const long long t0 = clock64();                                                               \
    asm volatile(body                                                                             \
                 :                                                                                \
                 : "v"(own), "v"(first)                                                           \
                 : "v10", "v11", "v12", "v13", "v14", "v15", "v16", "v17", "s40", "s41", "s42",  \
                   "s43", "s44", "s45", "s46", "s47", "vcc", "memory");                           \
    const long long t1 = clock64();                                                               \
    if (threadIdx.x == 0) out[idx] = t1 - t0;                                                     \
  }

__global__ void __launch_bounds__(kWave) issue_probe_kernel(long long* __restrict__ out) {
  __shared__ float lds[256];
  for (int i = threadIdx.x; i < 256; i += kWave) lds[i] = 0.f;
  __syncthreads();
  const unsigned own = (unsigned)(size_t)&lds[threadIdx.x], first = (unsigned)(size_t)&lds[0];
  // ordinary values in the registers the patterns compute on (nothing depends on their surviving)
  asm volatile(
      "v_mov_b32 v10, 1.0\n v_mov_b32 v11, 1.0\n v_mov_b32 v12, 1.0\n v_mov_b32 v13, 1.0\n"
      " v_mov_b32 v14, 1.0\n v_mov_b32 v15, 1.0\n v_mov_b32 v16, 1.0\n v_mov_b32 v17, 1.0\n"
      " s_mov_b32 s40, 1\n s_mov_b32 s41, 1\n s_mov_b32 s42, 1\n s_mov_b32 s43, 1"
      :
      :
      : "v10", "v11", "v12", "v13", "v14", "v15", "v16", "v17", "s40", "s41", "s42", "s43");
  for (int rep = 0; rep < 2; ++rep) {  // (the second pass runs from a warm instruction cache)
  MPL_ISSUE_TIMED(0, "")
  MPL_ISSUE_TIMED(1, ".rept 120\n v_add_f32 v10, v10, v14\n v_add_f32 v11, v11, v14\n v_add_f32 v12, v12, v14\n v_add_f32 v13, v13, v14\n .endr")
  MPL_ISSUE_TIMED(2, ".rept 480\n v_add_f32 v10, v10, v14\n .endr")
  MPL_ISSUE_TIMED(3, ".rept 480\n v_fmac_f32 v11, v12, v13\n .endr")
  MPL_ISSUE_TIMED(4, ".rept 480\n v_fma_f32 v10, v11, v12, v13\n .endr")
  MPL_ISSUE_TIMED(5, ".rept 480\n v_fma_f32 v10, v11, v12, s40\n .endr")
  MPL_ISSUE_TIMED(6, ".rept 480\n v_min3_f32 v10, v11, v12, v13\n .endr")
  MPL_ISSUE_TIMED(7, ".rept 480\n v_cmp_eq_f32_e64 s[44:45], v10, v15\n .endr")
  MPL_ISSUE_TIMED(8, ".rept 480\n v_cndmask_b32_e64 v10, v11, v12, s[40:41]\n .endr")
  MPL_ISSUE_TIMED(9, ".rept 480\n v_cndmask_b32_e64 v10, v10, 3, s[40:41]\n .endr")
  MPL_ISSUE_TIMED(10, ".rept 160\n v_cmp_eq_f32_e32 vcc, v10, v14\n s_nop 1\n v_cndmask_b32_e32 v16, 3, v16, vcc\n .endr")
  MPL_ISSUE_TIMED(11, ".rept 120\n v_cmp_eq_f32_e64 s[44:45], v10, v14\n v_cmp_eq_f32_e64 s[46:47], v11, v14\n v_cndmask_b32_e64 v16, v16, 3, s[44:45]\n v_cndmask_b32_e64 v17, v17, 4, s[46:47]\n .endr")
  MPL_ISSUE_TIMED(12, ".rept 480\n s_nop 0\n .endr")
  MPL_ISSUE_TIMED(13, ".rept 480\n s_nop 1\n .endr")
  MPL_ISSUE_TIMED(14, ".rept 480\n s_add_i32 s44, s40, 1\n .endr")
  MPL_ISSUE_TIMED(15, ".rept 480\n v_readlane_b32 s44, v10, 3\n .endr")
  MPL_ISSUE_TIMED(16, ".rept 240\n s_nop 1\n v_min_f32_dpp v10, v10, v10 row_shr:1 row_mask:0xf bank_mask:0xf\n .endr")
  MPL_ISSUE_TIMED(17, ".rept 160\n v_min_f32_dpp v10, v10, v10 row_shr:1 row_mask:0xf bank_mask:0xf\n v_add_f32 v11, v11, v14\n v_add_f32 v12, v12, v14\n .endr")
  MPL_ISSUE_TIMED(18, ".rept 480\n v_exp_f32 v10, v15\n .endr")
  MPL_ISSUE_TIMED(19, ".rept 480\n v_rcp_f32 v10, v15\n .endr")
  MPL_ISSUE_TIMED(20, ".rept 53\n ds_bpermute_b32 v10, %0, v15\n ds_bpermute_b32 v11, %0, v15\n ds_bpermute_b32 v12, %0, v15\n ds_bpermute_b32 v13, %0, v15\n ds_bpermute_b32 v10, %0, v15\n ds_bpermute_b32 v11, %0, v15\n ds_bpermute_b32 v12, %0, v15\n ds_bpermute_b32 v13, %0, v15\n s_waitcnt lgkmcnt(0)\n .endr")
  MPL_ISSUE_TIMED(21, ".rept 240\n ds_bpermute_b32 v10, %0, v15\n s_waitcnt lgkmcnt(0)\n .endr")
  MPL_ISSUE_TIMED(22, ".rept 240\n ds_read_b32 v10, %0\n s_waitcnt lgkmcnt(0)\n .endr")
  MPL_ISSUE_TIMED(23, ".rept 160\n ds_add_f32 %0, v15\n ds_wrxchg_rtn_b32 v10, %0, %1\n s_waitcnt lgkmcnt(0)\n .endr")
  MPL_ISSUE_TIMED(24, ".rept 240\n ds_add_f32 %1, v15\n s_waitcnt lgkmcnt(0)\n .endr")
  }
}
#undef MPL_ISSUE_TIMED

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
  if (wave_min_fast(y) != 0.f) ok = 0;
  for (int special = 0; special < 64; special += 7)
    if (wave_min_fast(y + (lane == special ? -100.f : 0.f)) != (float)((special * 37 + 11) % 64) - 100.f)
      ok = 0;
  if (wave_min_fast(lane < 21 ? (float)(30 - lane) : INFINITY) != 10.f) ok = 0;
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

}  // namespace

extern "C" {

const char* mplp_last_error(void) { return g_probe_err; }

int mplp_selftest_wave_ops(int* out, void* stream) {
  if (out == nullptr) return pfail(kEinval, "selftest: null pointer");
  selftest_kernel<<<1, kWave, 0, (hipStream_t)stream>>>(out);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return pfail(kElaunch, "selftest: %s", hipGetErrorString(e));
  return 0;
}


int mplp_copy(int shape, int n_in, int n_out, const float* in, float* out, int height,
                   int width, int n_labels, void* stream) {
  if (in == nullptr || out == nullptr) return pfail(kEinval, "probe_copy: null pointer");
  if (shape < 0 || shape > MPLP_STREAM) return pfail(kEinval, "probe_copy: unknown shape");
  if (height < 1 || width < 1 || n_labels < 4 || n_labels > 256 || (n_labels & 3))
    return pfail(kEinval, "probe_copy: n_labels must be a multiple of 4 in [4, 256]");
  if ((int64_t)height * width * n_labels / 4 / 256 > 0x7fffffff)
    return pfail(kEinval, "probe_copy: plane too large");
  hipStream_t st = (hipStream_t)stream;
  const int key = n_in * 10 + n_out;
  switch (key) {
    case 11: launch_probe<1, 1>(shape, in, out, height, width, n_labels, st); break;
    case 13: launch_probe<1, 3>(shape, in, out, height, width, n_labels, st); break;
    case 30: launch_probe<3, 0>(shape, in, out, height, width, n_labels, st); break;
    case 32: launch_probe<3, 2>(shape, in, out, height, width, n_labels, st); break;
    case 43: launch_probe<4, 3>(shape, in, out, height, width, n_labels, st); break;
    default:
      return pfail(kEinval, "probe_copy: (n_in, n_out) must be one of (1,1) (1,3) (3,0) (3,2) (4,3)");
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return pfail(kElaunch, "probe_copy: %s", hipGetErrorString(e));
  return 0;
}

int mplp_issue_count(void) { return kNumIssuePatterns; }

const char* mplp_issue_name(int pattern) {
  return pattern >= 0 && pattern < kNumIssuePatterns ? kIssuePatterns[pattern].name : "";
}

int mplp_issue_slots(int pattern) {
  return pattern >= 0 && pattern < kNumIssuePatterns ? kIssuePatterns[pattern].slots : -1;
}

int mplp_issue(long long* clocks, int n, void* stream) {
  if (clocks == nullptr) return pfail(kEinval, "probe_issue: null pointer");
  if (n < kNumIssuePatterns) return pfail(kEinval, "probe_issue: room for %d results needed", kNumIssuePatterns);
  issue_probe_kernel<<<1, kWave, 0, (hipStream_t)stream>>>(clocks);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return pfail(kElaunch, "probe_issue: %s", hipGetErrorString(e));
  return 0;
}

}  // extern "C"
