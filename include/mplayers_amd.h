/*
 * C ABI of libmplayers_hip.so: min-sum message passing (TRWP, ISGMR) on grid MRFs for gfx950.
 *
 * Every pointer is a DEVICE pointer unless said otherwise (the mpl_*_forward_cpu calls take host
 * pointers); all tensors are contiguous with the
 * label axis innermost.  The caller owns and allocates every buffer, exactly as the reference's
 * operators require (pytorch/MP_module.py:26-50, 65-78); buffers marked "zero-filled" must come
 * in zeroed, as the reference's caller provides them.  `stream` is a hipStream_t (NULL = the
 * default stream).  Nothing here allocates device memory, and nothing but mpl_profile_end(), which
 * waits for the events of its bracket, synchronises with the host.
 *
 * Shapes:  B = batch * n_cv,  P = B*H*W pixels,  N = P*L.
 *   unary, cost_final, unary_update, dcost_final, dunary, dunary_update   (B, H, W, L)  fp32
 *   msg, msg_update, dmsg, dmsg_update                                    (n_dir, B, H, W, L) fp32
 *   edge_weights, dedge_weights                                           (n_dir, B, H, W) fp32
 *   msg_min_index   (n_iter, n_dir, B, H, W, L) uint8      msg_norm_index (n_iter, n_dir, B, H, W) uint8
 *   label_all       (n_iter, B, H, W) uint8
 *   context         ctx2d ? (L, L), entries [min(a,b)*L + max(a,b)] read : >= L floats, [|a-b|] read
 *   dcontext        same shape as context (zero-filled; only off-diagonal / k>=1 entries are written,
 *                   unless MPL_F_DCONTEXT_SAME_LABEL is given)
 *
 * Return value: 0 on success, a negative MPL_E* code otherwise; mpl_last_error() then returns a
 * message for the calling thread.  On error nothing has been launched.
 */
#ifndef MPLAYERS_AMD_H_
#define MPLAYERS_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MPL_OK 0
#define MPL_EINVAL (-1)   /* bad shape / null pointer / unsupported size */
#define MPL_ELAUNCH (-2)  /* the HIP runtime refused a launch */

#define MPL_MAX_LABELS 256 /* argmin indices are uint8 (reference: MAX_DISPARITY, MPLayers/setup.py:58) */
#define MPL_MAX_DIRS 16    /* direction table of MPLayers/common.cpp:28-76 */

typedef struct mpl_shape {
  int n_dir;  /* 2..16, even: direction d pairs with d^1 (common.cpp:23-26) */
  int batch;  /* batch * n_cv */
  int height;
  int width;
  int n_disp; /* labels, <= MPL_MAX_LABELS */
  int ctx2d;  /* 1: (L,L) context table (the reference selects it by n_disp == 21); needs L <= 64 */
} mpl_shape;

/* Per-call flags, the `flags` argument of the forward and backward entry points (no counterpart in
 * the reference).  0 is the reference's contract with the process defaults of mpl_set_option().
 * A flag a call has no use for is ignored; unknown bits are rejected with MPL_EINVAL. */
#define MPL_F_MSG_UNINIT 0x01u
/* forward calls.  Without it `msg` holds the initial messages (the reference's contract: the
 * caller zero-fills it).  With it the contents of `msg` on entry are ignored: the messages start at
 * zero and the library writes every element itself, which saves the caller's memset and the passes
 * that would read the zeros back. */
#define MPL_F_PACKED_OFF 0x02u
#define MPL_F_PACKED_ALWAYS 0x04u
/* scans of at most 32 labels with several chains per wavefront: never / whenever the label count
 * allows it, for this call (neither bit: the process default, see MPL_OPT_PACKED_SCANS). */
#define MPL_F_FUSED_U_OFF 0x08u
/* ISGMR forward: always run the pass that stores U (see MPL_OPT_FUSED_U). */
#define MPL_F_DCONTEXT_SAME_LABEL 0x10u
/* hard backward calls: dcontext also collects the pairs whose front label equals their own label
 * (entry 0 of a 1-D table, the diagonal of a 2-D one), as the hard operator of the reference's
 * TRWP_hard_soft build does (MPLayers/TRWP_hard_soft/TRWP_backward.cu:104-111, 188-195, 258-265);
 * the TRWP and ISGMR builds skip them (MPLayers/TRWP/TRWP_backward.cu:111-112). */
#define MPL_F_FUSED_PAIRS_OFF 0x20u
/* TRWP calls: one launch per direction even where a launch has so few chains (at most one per
 * SIMD of the device) that the library would run both sweeps of a pair of opposite directions in
 * one. */
#define MPL_F_DENSE_TABLE 0x40u
/* forward calls: the caller declares that its 1-D pairwise table is dense (a learned table, an
 * untruncated one): no constant tail that the O(L) band scan could use, so the scans take their
 * O(L^2) step.  With more than 64 labels, launches of at most one and a half chains per SIMD then
 * put four or two wavefronts on every chain, each scanning a share of the front labels of a pixel.
 * The kind of the table is otherwise only known on the device, after the launch is sized.  The
 * launches that get several wavefronts per chain take the dense step whatever the table: a band
 * table (a constant tail from entry 32 at the latest) then runs slower and gives the same bits as
 * without the flag; a wider truncated linear table loses its O(L) label scan, whose values may
 * differ from the dense step's in the last bits where the table is not integer-valued, both within
 * the tolerance of the parity tests. */
#define MPL_F_ALL 0x7fu

/* Replaces lib_*.TRWP.forward: MPLayers/TRWP/TRWP.cpp:245-283 (Forward) -> TRWP_forward.cu:378-560.
 * msg: initial messages in, final normalised messages out.  msg_min_index/msg_norm_index NULL =>
 * inference (no index stores).  label_all NULL => no per-iteration labels.  unary_update: scratch
 * plane (carries the running belief during the call).  cost_final doubles as scratch until the final aggregation. */
int mpl_trwp_forward(const mpl_shape* shape, unsigned flags, float rho, int n_iter,
                     int enable_min_a_dir, const float* unary, const float* context,
                     const float* edge_weights, float* msg, float* cost_final,
                     uint8_t* msg_min_index, uint8_t* msg_norm_index, float* unary_update,
                     uint8_t* label_all, void* stream);

/* Replaces lib_*.TRWP.backward: MPLayers/TRWP/TRWP.cpp:285-318 -> TRWP_backward.cu:277-433.
 * dunary receives the gradient; dcontext and dedge_weights (zero-filled) accumulate; dmsg is
 * scratch (n_dir planes, any contents); dunary_update is accepted and unused.
 * dcontext and / or dedge_weights may be NULL when the caller has no use for that gradient (a fixed
 * pairwise table, edge weights that are not learned): the reverse scans then leave that part of
 * their step out; dunary is the same bit for bit. */
int mpl_trwp_backward(const mpl_shape* shape, unsigned flags, float rho, int n_iter,
                      const float* context, const float* edge_weights, const float* dcost_final,
                      const uint8_t* msg_min_index, const uint8_t* msg_norm_index, float* dunary,
                      float* dcontext, float* dedge_weights, float* dmsg, float* dunary_update,
                      void* stream);

/* Replaces lib_*.ISGMR.forward: MPLayers/ISGMR/ISGMR.cpp:300-342 -> ISGMR_forward.cu:433-665.
 * msg_update: second message buffer (any contents); on return msg holds the final messages,
 * msg_update intermediate values; unary_update is accepted and unused. */
int mpl_isgmr_forward(const mpl_shape* shape, unsigned flags, int enable_sgm, float rho,
                      int n_iter, int enable_min_a_dir, const float* unary, const float* context,
                      const float* edge_weights, float* msg, float* cost_final,
                      uint8_t* msg_min_index, uint8_t* msg_norm_index, float* unary_update,
                      float* msg_update, uint8_t* label_all, void* stream);

/* Replaces lib_*.ISGMR.backward: MPLayers/ISGMR/ISGMR.cpp:344-379 -> ISGMR_backward.cu:290-493.
 * dmsg_update and dmsg are scratch (n_dir planes each, any contents); dmsg may be NULL (the pass
 * then works in place in dmsg_update and moves somewhat more data); dunary_update is unused.
 * dcontext and / or dedge_weights may be NULL, as for mpl_trwp_backward. */
int mpl_isgmr_backward(const mpl_shape* shape, unsigned flags, int enable_sgm, float rho,
                       int n_iter, const float* context, const float* edge_weights,
                       const float* dcost_final, const uint8_t* msg_min_index,
                       const uint8_t* msg_norm_index, float* dunary, float* dcontext,
                       float* dedge_weights, float* dmsg, float* dunary_update,
                       float* dmsg_update, void* stream);

/* The CPU branch of lib_*.TRWP.forward and lib_*.ISGMR.forward: what the reference's operators run
 * when their tensors are not on the GPU (ForwardCPU, MPLayers/TRWP/TRWP.cpp:172-243 reached from
 * :275-282, MPLayers/ISGMR/ISGMR.cpp:190-298 reached from :330-339).  HOST pointers; the calls run
 * on the calling thread and on up to MPL_OPT_CPU_THREADS worker threads and return when done.
 * That path has its own semantics, reproduced bit for bit: forward only, every edge weight 1, no
 * argmin indices; the pairwise table of direction d is read at context + d * n_disp * n_disp, so
 * `context` holds (n_dir - 1) * n_disp^2 floats plus one table (n_disp^2 with ctx2d, else n_disp);
 * value = rho * (unary + sum_k m_k) - m_inv + ctx in that order; labels are 0 for 256 labels
 * (the reference's unsigned char loop counter, common.cpp:152).  label_all may be NULL.
 * mpl_isgmr_forward_cpu with enable_sgm REPLACES `unary` by the sum of the new messages after every
 * iteration and clears `msg` (ISGMR.cpp:255-261): unary is an in/out tensor there.  msg_update is
 * the second message buffer (zero-filled by the caller, as `msg`).  There is no CPU backward
 * (TRWP.cpp:315-316). */
int mpl_trwp_forward_cpu(const mpl_shape* shape, float rho, int n_iter, const float* unary,
                         const float* context, float* msg, float* cost_final, uint8_t* label_all);
int mpl_isgmr_forward_cpu(const mpl_shape* shape, int enable_sgm, float rho, int n_iter,
                          float* unary, const float* context, float* msg, float* cost_final,
                          float* msg_update, uint8_t* label_all);

/* Soft-weighted TRWP: replaces lib_*.TRWP_hard_soft.forward_soft, MPLayers/TRWP_hard_soft/TRWP.cpp:
 * 313-349 (ForwardSoft) -> TRWP_forward_soft.cu:378-559.  The min over front labels becomes the
 * expectation of the dual under softmin weights.  n_disp <= MPL_MAX_LABELS as for the reference's
 * stereo build (TRWP.cpp:336-340); 2-D context tables up to 64 labels.
 *   msg_edge_label (n_iter, n_dir, B, H, W, L, L) fp32: every dual of every pixel, kept for the
 *   backward pass (even directions [fd][cd], odd ones [cd][fd]); blocks of chain-start pixels are
 *   not written.  NULL together with msg_norm_index => inference. */
int mpl_trwp_soft_forward(const mpl_shape* shape, unsigned flags, float rho, int n_iter,
                          const float* unary, const float* context, const float* edge_weights,
                          float* msg, float* msg_edge_label, uint8_t* msg_norm_index,
                          float* cost_final, float* unary_update, uint8_t* label_all,
                          void* stream);

/* Replaces lib_*.TRWP_hard_soft.backward_soft, TRWP.cpp:351-383 (BackwardSoft) ->
 * TRWP_backward_soft.cu:422-548.  dcontext also receives the zero-offset / diagonal terms here
 * (the hard operator skips them).  dmsg is scratch (n_dir planes, any contents). */
int mpl_trwp_soft_backward(const mpl_shape* shape, unsigned flags, float rho, int n_iter,
                           const float* dcost_final, const float* context,
                           const float* edge_weights, const float* msg_edge_label,
                           const uint8_t* msg_norm_index, float* dunary, float* dcontext,
                           float* dedge_weights, float* dmsg, float* dunary_update, void* stream);

/* Stand-alone softmin of stored blocks: replaces lib_*.TRWP_hard_soft.soft_weighted_message and
 * soft_weighted_message_back, TRWP.cpp:385-417 -> TRWP_swbp.cu:131-321.  message (n_trees, L, L)
 * laid out [fd][cd]; message_soft_sum_norm (n_trees, L) = sum_fd softmax_fd(-message) * message,
 * minus its minimum over cd; message_soft_sum_min_ind (n_trees) uint8: the label of that minimum
 * (largest on ties).  The backward call fills dmessage (n_trees, L, L). */
int mpl_soft_weighted_message(int n_trees, int n_disp, const float* message,
                              float* message_soft_sum_norm, uint8_t* message_soft_sum_min_ind,
                              void* stream);
int mpl_soft_weighted_message_back(int n_trees, int n_disp, const float* dmessage_soft_sum_norm,
                                   const float* message, const uint8_t* message_soft_sum_min_ind,
                                   float* dmessage, void* stream);

/* Per-kernel timing for benchmarks (no counterpart in the reference, which times whole calls with
 * time.time(), MPLayers/main.py:271-313).  Between mpl_profile_begin() and mpl_profile_end() every
 * kernel launch of this library is bracketed by HIP events on its own stream; mpl_profile_end()
 * waits for them and fills stats[kind] for kind < n_stats.  Events cost a few microseconds per
 * launch; nothing is recorded outside such a bracket.  One bracket at a time per process: the
 * bracket is process-wide state (calls on any thread and stream between begin and end are
 * recorded into it), so a second begin before the end restarts it. */
#define MPL_KERNEL_FWD_SWEEP 0      /* forward scan of one direction (TRWP) */
#define MPL_KERNEL_BWD_SWEEP 1      /* reverse scan of one direction (TRWP) */
#define MPL_KERNEL_BELIEF 2         /* S = unary + sum of messages (TRWP, once per call) */
#define MPL_KERNEL_AGGREGATE 3      /* cost_final */
#define MPL_KERNEL_LABEL 4          /* per-iteration labels */
#define MPL_KERNEL_COMBINE 5        /* ISGMR backward: per-iteration gradient recombination */
#define MPL_KERNEL_OTHER 6
#define MPL_KERNEL_FWD_SWEEP_ALL 7  /* forward scan of all directions in one launch (ISGMR) */
#define MPL_KERNEL_BWD_SWEEP_ALL 8  /* reverse scan of all directions in one launch (ISGMR) */
#define MPL_KERNEL_UNARY_ALL 9     /* ISGMR forward: per-iteration U of every direction */
#define MPL_KERNEL_KINDS 10
typedef struct mpl_kernel_stat {
  int launches;
  double total_ms;
} mpl_kernel_stat;
int mpl_profile_begin(void);
int mpl_profile_end(mpl_kernel_stat* stats, int n_stats);

/* Number of chains of direction `dir` (0..15) on an H x W grid: the reference's n_trees
 * (common.cpp:78-87) for images of at least 2 x 2 pixels (on thinner images the reference also
 * counts trees of the two-pixel steps that never enter the image).  Host-only helper; -1 for a
 * direction outside the table. */
int mpl_n_chains(int dir, int height, int width);

/* Whether the forward scans take their O(L^2) step on the 1-D pairwise table `context` (n_disp
 * floats in HOST memory): 1 when it has neither a constant tail from entry 32 at the latest with no
 * entry above the tail (the band scan) nor the shape c[k] = min(c[1] * k, c[n_disp - 1]) with
 * c[0] = 0 (the label scan of a truncated linear table), else 0; -1 for a NULL table or n_disp < 1.
 * It is what a caller who builds its table on the host passes on as MPL_F_DENSE_TABLE; the library
 * itself looks at the table on the device, after its launches are sized.  Host-only helper, no
 * counterpart in the reference. */
int mpl_table_is_dense(const float* context, int n_disp);

/* Edge-weight producer, the layer's immediate upstream: replaces getEdgeShift of
 * utils/edge_weights.py:45-111.  image (batch, channels, H, W) fp32 -> out (n_dirs, batch, channels,
 * H, W) fp32, fully written: for direction d with step r_d and every pixel p whose front neighbour
 * q = p - r_d is inside the image, out[d, p] = f_mode(|I(p) - I(q)|); 0 where q is outside.
 * The channel-reducing modes (SUPERPIXEL, CUE_REAL, CUE_BINARY, THRESHOLD) take batch == 1 and
 * write their per-pixel value to every channel plane, as the reference's broadcasting assignment
 * does for one image.  dir_sums: 16 doubles of device scratch, used by CUE_BINARY only (may be
 * NULL otherwise).  Modes are the reference's edge_mode strings: */
#define MPL_EDGE_GT 0          /* 'gt_edge': 1 where equal and the pixel is not 255, else 0 */
#define MPL_EDGE_SUPERPIXEL 1  /* 'superpixel_edge': 1 where all channels are equal */
#define MPL_EDGE_LINEAR 2      /* 'sobel', 'edge_net_sigmoid': 1 - diff */
#define MPL_EDGE_CANNY 3       /* 'canny': 1 - diff, diff forced to 1 on edge pixels (value 1) */
#define MPL_EDGE_EXP 4         /* 'edge_net': exp(-diff) */
#define MPL_EDGE_CUE_REAL 5    /* 'kernel_cue_real': exp(-mean_c(diff^2) / (2 sigma^2)) */
#define MPL_EDGE_CUE_BINARY 6  /* 'kernel_cue_binary': CUE_REAL >= 0.8 * its mean over valid pixels */
#define MPL_EDGE_THRESHOLD 7   /* 'threshold': penalty where mean_c(diff^2) < threshold, else 0 */
#define MPL_EDGE_SHIFT 8       /* any other string: the front neighbour's value I(q) */
#define MPL_EDGE_MODES 9
int mpl_edge_shift(int mode, const float* image, int batch, int channels, int height, int width,
                   int n_dirs, float sigma, float threshold, float penalty, float* out,
                   double* dir_sums, void* stream);

/* mpl_edge_shift for callers that cannot allocate or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results as mpl_edge_shift without dir_sums: the per-direction
 * sums of CUE_BINARY live in a static device array of the library (MPL_MAX_DIRS doubles, 128
 * bytes on every GPU the library runs on, held until the process ends), whose address is resolved
 * on the first call on a device.  The call allocates nothing; n_dirs beyond MPL_MAX_DIRS is refused
 * with MPL_EINVAL.  All calls on one GPU share that array (it is cleared by a kernel at the start
 * of each call): calls that overlap on one GPU, on different streams, race. */
int mpl_edge_shift_static(int mode, const float* image, int batch, int channels, int height,
                          int width, int n_dirs, float sigma, float threshold, float penalty,
                          float* out, void* stream);

/* Stereo data term, the layers' upstream in the reference's energy-minimisation driver: replaces
 * computeDSI (MPLayers/aux/aux.cpp:5-98) as called by compute_all_terms
 * (MPLayers/aux/auxPy.cpp:22,62-66: birchfield = 1, squared_diffs = 0, trunc_diffs = 255).
 * left/right: device images, (H, W, bands) uint8, interleaved; the first min(3, bands) bands are
 * compared.  data_cost (H, W, n_labels) fp32, fully written: the matching cost of pixel (y, x)
 * with (y, x - d) of the right image, summed over the colour bands and truncated at
 * colours * |trunc_diffs| (trunc_diffs^2 for squared differences); matches outside the image cost
 * min(colours * 255 [* 255], truncation).  Integer arithmetic, exact. */
int mpl_stereo_data_cost(const uint8_t* left, const uint8_t* right, int height, int width,
                         int bands, int n_labels, int birchfield, int squared_diffs,
                         int trunc_diffs, float* data_cost, void* stream);

/* Gradient cues of the same driver: replaces computeCues (MPLayers/aux/aux.cpp:100-170) and the
 * re-packing of MPLayers/aux/auxPy.cpp:83-99.  h_cue (H, W-1) and v_cue (W, H-1) fp32 hold
 * grad_penalty where the summed squared colour difference to the right / lower neighbour is below
 * colours * grad_thresh^2, else 1. */
int mpl_gradient_cues(const uint8_t* image, int height, int width, int bands, int grad_thresh,
                      float grad_penalty, float* h_cue, float* v_cue, void* stream);

/* Energy of labellings, the layers' downstream in the same driver: replaces calEnergy
 * (tools/matlab/MRF/calEnergy.m:2-48), generalised from the 4-connected grid to the layers'
 * direction table and to their edge weights.  labels (n_labelings, batch, H, W) uint8 (for
 * instance the label_all output of a forward call); unary, context, edge_weights (may be NULL:
 * all ones) as in mpl_trwp_forward.  energy (n_labelings, 2) fp64, overwritten:
 *   energy[i][0] = sum_p unary[p, x_p]
 *   energy[i][1] = sum over even directions d and pixels p with q = p - r_d inside the image of
 *                  edge_weights[d, p] * ctx(x_p, x_q)          (every undirected edge once)
 * accumulated in fp64 with atomics (the order of the partial sums is not fixed). */
int mpl_mrf_energy(const mpl_shape* shape, int n_labelings, const float* unary,
                   const float* context, const float* edge_weights, const uint8_t* labels,
                   double* energy, void* stream);

/* Batched 2-D transpose src (batch, rows, cols) -> dst (batch, cols, rows), fp32: the layout change
 * between the network's (batch, labels, H, W) tensors and the kernels' (batch, H, W, labels), which
 * the reference's module does with permute().contiguous() (pytorch/MP_module.py:199,203,233).
 * rows = labels, cols = H*W on the way in; rows = H*W, cols = labels on the way out. */
int mpl_transpose(const float* src, float* dst, int batch, int64_t rows, int64_t cols,
                  void* stream);

/* Message of the last failed call on this thread ("" if none). */
const char* mpl_last_error(void);

/* Process-wide defaults of what the per-call flags MPL_F_PACKED_* and MPL_F_FUSED_U_OFF select
 * (no counterpart in the reference).  A call that passes one of those flags is not affected by
 * these; the values are read atomically once per call.
 * MPL_OPT_PACKED_SCANS (default 1): launches with a 2-D table of at most 32 labels and more
 * chains than the device has SIMDs (four per compute unit; twice as many with 21 labels), and
 * launches with a 1-D table of at most 8 labels and more than 6 chains per SIMD or of at most 16
 * labels and more than 9, whose planes stay below 2 GiB, are scanned with several chains per
 * wavefront (on an MI355X, 1024 SIMDs: more than 1024 / 2048 / 6144 / 9216 chains); 0
 * forces the one-chain-per-wavefront kernels, 2 packs whenever the label count (at most 32) allows
 * it.  The packed step scans every front label whatever the table, so it is not the default for
 * 1-D tables, which are nearly always bands; a caller whose 1-D tables of up to 32 labels are dense
 * and whose launches have thousands of chains gains from 2 (or MPL_F_PACKED_ALWAYS per call).  The
 * results agree to the parity tolerance in every case. */
#define MPL_OPT_PACKED_SCANS 0
/* MPL_OPT_FUSED_U (default 1): ISGMR forward with 4 directions, rho == 1 and one chain per
 * wavefront (more than 32 labels, or a launch the packed scans do not take) forms U inside the scans (unary + the old messages of the other pair of directions) instead of
 * storing it in a pass of its own; 0 always runs that pass (results agree to the parity tolerance,
 * bit for bit on inputs whose sums do not round). */
#define MPL_OPT_FUSED_U 1
/* MPL_OPT_BELIEF_REBUILD (default MPL_BELIEF_REBUILD_DEFAULT): the TRWP forward calls, hard and
 * soft-weighted, keep unary + the sum of all messages as a plane that every sweep updates by
 * differences, where the reference re-sums it before every sweep (TRWP_forward.cu:60-80).  Every
 * `value` iterations the plane is re-summed from the messages as the reference sums them, so the
 * rounding of at most that many iterations' updates is ever in it; 0: never; -1: the library
 * chooses (calls of at most 64 direction sweeps, n_iter * n_dir, are not re-summed; longer ones
 * every max(1, 32 / n_dir) iterations). */
#define MPL_OPT_BELIEF_REBUILD 2
#define MPL_BELIEF_REBUILD_DEFAULT (-1)
/* MPL_OPT_CPU_THREADS (default 0: 16, the reference's NUM_THREADS, tools/cpp/utils.h:17): threads
 * the mpl_*_forward_cpu calls spread their chains over. */
#define MPL_OPT_CPU_THREADS 3
/* MPL_OPT_DENSE_SPLIT_WAVES (default 0: the library chooses per launch): wavefronts per chain of
 * the forward launches that MPL_F_DENSE_TABLE splits, at most 8 and at most what leaves every
 * wavefront a front label (1: never split).  For tests and measurements. */
#define MPL_OPT_DENSE_SPLIT_WAVES 4
int mpl_set_option(int option, int value);

/* Library version: major * 100 + minor. */
int mpl_version(void);

#ifdef __cplusplus
}
#endif

#endif /* MPLAYERS_AMD_H_ */
