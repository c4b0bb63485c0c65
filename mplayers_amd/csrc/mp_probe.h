/*
 * C ABI of libmplayers_probe.so: measurement tools of the benchmark and the tests, built from
 * mp_probe.hip next to the product library.  Nothing here is an operator and nothing here has a
 * counterpart in the reference; libmplayers_hip.so neither contains nor needs any of it.
 * Pointers are device pointers; `stream` is a hipStream_t (NULL: the default stream).  The calls
 * only launch kernels: no allocation, no synchronisation.  0 on success, a negative code
 * otherwise; mplp_last_error() then returns a message for the calling thread.
 */
#ifndef MPLAYERS_AMD_MP_PROBE_H_
#define MPLAYERS_AMD_MP_PROBE_H_

#ifdef __cplusplus
extern "C" {
#endif

/* Bandwidth probe: moves n_in planes of (height, width, n_labels) fp32 from `in` to n_out planes at
 * `out` (sum of the inputs, + k for plane k) in the scans' access shape -- one long-lived
 * wavefront per row (MPLP_ROWS) or per column (MPLP_COLUMNS), one pixel vector per step, eight
 * pixels in flight -- or as a one-pass streaming kernel (MPLP_STREAM).  `in` holds n_in planes,
 * `out` max(n_out, 1); (n_in, n_out) is one of (1,1) (1,3) (3,0) (3,2) (4,3); n_labels a multiple
 * of 4. */
#define MPLP_ROWS 0
#define MPLP_COLUMNS 1
#define MPLP_STREAM 2
int mplp_copy(int shape, int n_in, int n_out, const float* in, float* out, int height, int width,
              int n_labels, void* stream);

/* Issue probe: one wavefront, alone on its SIMD, runs a few hundred copies of each of
 * mplp_issue_count() instruction patterns between two reads of the shader clock and stores the
 * elapsed clocks of pattern i in clocks[i] (room for n >= mplp_issue_count() values; pattern 0 is
 * an empty region, the overhead of the two reads).  mplp_issue_slots(i) is the number of issue
 * slots pattern i was run for, idle slots included, mplp_issue_name(i) what it is.  The scans of
 * launches with fewer chains than the chip has SIMDs are bound by these costs. */
int mplp_issue_count(void);
const char* mplp_issue_name(int pattern);
int mplp_issue_slots(int pattern);
int mplp_issue(long long* clocks, int n, void* stream);

/* Check of the wavefront primitives the scan kernels are built on (cross-lane shifts, min / sum
 * reductions, ballots), on the device that runs them.  out: 8 ints of device memory;
 * out[0] == 1 once the kernel has run and every check passed, out[1..2] the lanes that passed. */
int mplp_selftest_wave_ops(int* out, void* stream);

const char* mplp_last_error(void);

#ifdef __cplusplus
}
#endif

#endif /* MPLAYERS_AMD_MP_PROBE_H_ */
