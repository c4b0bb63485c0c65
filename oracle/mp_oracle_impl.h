/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's min-sum message
 * passing (TRWP / ISGMR) with the semantics of its GPU kernels: per-pixel edge
 * weights, argmin indices, tie rules and the backward pass.  Nothing in the
 * product path may call into this file.
 *
 * The file is included twice by mp_oracle.c, once with REAL=float (bit-level
 * comparisons of values and indices) and once with REAL=double (gradient checks).
 * Every function cites the reference file:line it follows.  Offsets are 64-bit
 * (the reference uses 32-bit `uint` offsets, which overflow for large volumes).
 *
 * Layouts (all contiguous, label innermost):
 *   unary, cost_final        (B, H, W, L)          B = batch * n_cv
 *   msg                      (n_dir, B, H, W, L)
 *   edge_weights             (n_dir, B, H, W)      weight stored at the RECEIVING pixel
 *   msg_min_index            (n_iter, n_dir, B, H, W, L)  uint8
 *   msg_norm_index           (n_iter, n_dir, B, H, W)     uint8
 *   label_all                (n_iter, B, H, W)            uint8
 *   context                  (L, L) when ctx2d (only i<=j entries are read), else >= L floats
 */

#ifndef REAL
#error "include from mp_oracle.c"
#endif

/* ---- context lookup: TRWP_forward.cu:131-135 ------------------------------------ */
static inline int64_t FN(ctx_offset)(int L, int ctx2d, int cd, int fd) {
  if (ctx2d) {
    int lo = cd < fd ? cd : fd, hi = cd < fd ? fd : cd;
    return (int64_t)lo * L + hi;
  }
  return cd > fd ? cd - fd : fd - cd;
}

/* ---- UpdateUnaryKernel: TRWP_forward.cu:60-80, ISGMR_forward.cu:101-121 ---------- */
/* U = ((unary + m_0 + ... + m_{n-1}) - m_dir) * rho - m_inv, in that evaluation order */
static void FN(update_unary)(const mpo_geom* g, int dir, REAL rho, const REAL* unary,
                             const REAL* msg, REAL* U) {
  int64_t N = mpo_plane(g);
  int inv = dir ^ 1; /* common.cpp:23-26 */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) {
    REAL v = unary[i];
    for (int k = 0; k < g->n_dir; ++k) v += msg[(int64_t)k * N + i];
    v -= msg[(int64_t)dir * N + i];
    v *= rho;
    v -= msg[(int64_t)inv * N + i];
    U[i] = v;
  }
}

/* ---- one pixel of the scan kernels: TRWP_forward.cu:117-168 + commonCUDA.cuh:92-129 - */
/* prev: the "shared memory" vector; gap_* optional diagnostics (second best - best).   */
static void FN(pixel_step)(int L, int ctx2d, REAL rho, const REAL* Ufront, const REAL* context,
                           REAL w, REAL* prev, REAL* tmp, REAL* m_out, uint8_t* idx_min,
                           uint8_t* idx_norm, REAL* gap_min, REAL* gap_norm) {
  for (int cd = 0; cd < L; ++cd) {
    REAL best = 0, second = (REAL)INFINITY;
    int arg = 0;
    for (int fd = L - 1; fd >= 0; --fd) { /* descending + strict '<': largest fd wins ties */
      REAL cv = context[FN(ctx_offset)(L, ctx2d, cd, fd)];
      REAL mv = rho * prev[fd];
      REAL v = Ufront[fd] + mv + w * cv;
      if (fd == L - 1) {
        best = v;
        arg = fd;
      } else if (v < best) {
        second = best;
        best = v;
        arg = fd;
      } else if (v < second) {
        second = v;
      }
    }
    tmp[cd] = best;
    if (idx_min) idx_min[cd] = (uint8_t)arg;
    if (gap_min) gap_min[cd] = second - best;
  }
  /* MsgNormNaive: scan cd from L-1 down, strict '<' => largest cd wins ties */
  REAL nmin = tmp[L - 1], nsecond = (REAL)INFINITY;
  int narg = L - 1;
  for (int cd = L - 2; cd >= 0; --cd) {
    if (tmp[cd] < nmin) {
      nsecond = nmin;
      nmin = tmp[cd];
      narg = cd;
    } else if (tmp[cd] < nsecond) {
      nsecond = tmp[cd];
    }
  }
  for (int cd = 0; cd < L; ++cd) {
    prev[cd] = tmp[cd] - nmin;
    m_out[cd] = prev[cd];
  }
  if (idx_norm) *idx_norm = (uint8_t)narg;
  if (gap_norm) *gap_norm = nsecond - nmin;
}

/* ---- a whole direction sweep: Horizontal/DiagonalWide/DiagonalNarrow kernels -------- */
/* TRWP_forward.cu:82-376 (ISGMR_forward.cu:123-431 differ only in the output plane).   */
static void FN(sweep)(const mpo_geom* g, int dir, REAL rho, const REAL* U, const REAL* context,
                      const REAL* w_dir, REAL* m_out, uint8_t* idx_min, uint8_t* idx_norm,
                      REAL* gap_min, REAL* gap_norm) {
  int L = g->L, H = g->H, W = g->W;
  int hs, ws;
  mpo_dir_step(dir, &hs, &ws);
  int n_trees = mpo_n_trees(dir, H, W);
  /* chains ("trees", one block each in the reference) are independent: one thread per chain */
#pragma omp parallel
  {
    REAL* prev = (REAL*)malloc(sizeof(REAL) * L);
    REAL* tmp = (REAL*)malloc(sizeof(REAL) * L);
#pragma omp for collapse(2) schedule(dynamic, 4)
    for (int bv = 0; bv < g->B; ++bv) {
      for (int tree = 0; tree < n_trees; ++tree) {
        int64_t pix_base = (int64_t)bv * H * W;
        int h0, w0, n_roll;
        mpo_tree_start(dir, hs, ws, H, W, tree, &h0, &w0, &n_roll);
        for (int l = 0; l < L; ++l) prev[l] = 0; /* shared vector zeroed per block */
        for (int i = 0; i <= n_roll; ++i) {
          int ch = h0 + i * hs, cw = w0 + i * ws;
          int fh = ch - hs, fw = cw - ws;
          if (ch < 0 || ch >= H || cw < 0 || cw >= W || fh < 0 || fh >= H || fw < 0 || fw >= W)
            continue;
          int64_t pc = pix_base + (int64_t)ch * W + cw;
          int64_t pf = pix_base + (int64_t)fh * W + fw;
          FN(pixel_step)(L, g->ctx2d, rho, U + pf * L, context, w_dir[pc], prev, tmp,
                         m_out + pc * L, idx_min ? idx_min + pc * L : NULL,
                         idx_norm ? idx_norm + pc : NULL, gap_min ? gap_min + pc * L : NULL,
                         gap_norm ? gap_norm + pc : NULL);
        }
      }
    }
    free(prev);
    free(tmp);
  }
}

/* ---- CostAggregateKernel: TRWP_forward.cu:31-58, ISGMR_forward.cu:69-99 --------------- */
static void FN(cost_aggregate)(const mpo_geom* g, int enable_min_a_dir, REAL unary_factor,
                               const REAL* unary, const REAL* msg, REAL* cost) {
  int64_t N = mpo_plane(g);
  const REAL dir_weight = 1; /* param_list[0].dir_weight == hypot(0,1) */
  for (int64_t i = 0; i < N; ++i) {
    REAL v = unary[i] * unary_factor;
    if (enable_min_a_dir) {
      REAL mn = msg[i];
      for (int k = 1; k < g->n_dir; ++k) {
        REAL m = msg[(int64_t)k * N + i];
        if (m < mn) mn = m;
      }
      v += mn;
    } else {
      for (int k = 0; k < g->n_dir; ++k) v += msg[(int64_t)k * N + i] / dir_weight;
    }
    cost[i] = v;
  }
}

/* ---- CalLabelKernel: TRWP_forward.cu:8-29 (lowest label wins ties) ---------------------- */
/* gap (optional diagnostic): second smallest cost minus the smallest, per pixel               */
static void FN(cal_label)(const mpo_geom* g, const REAL* cost, uint8_t* label, REAL* gap) {
  int64_t P = mpo_pixels(g);
  for (int64_t p = 0; p < P; ++p) {
    REAL mn = cost[p * g->L], second = (REAL)INFINITY;
    int arg = 0;
    for (int l = 1; l < g->L; ++l) {
      REAL c = cost[p * g->L + l];
      if (c < mn) {
        second = mn;
        mn = c;
        arg = l;
      } else if (c < second) {
        second = c;
      }
    }
    label[p] = (uint8_t)arg;
    if (gap) gap[p] = second - mn;
  }
}

/* ---- TRWP ForwardCUDA: TRWP_forward.cu:378-560 (Gauss-Seidel over directions) ----------- */
int FN(mpo_trwp_forward)(const mpo_geom* g, REAL rho, int n_iter, int enable_min_a_dir,
                         const REAL* unary, const REAL* context, const REAL* edge_weights,
                         REAL* msg, REAL* cost_final, uint8_t* msg_min_index,
                         uint8_t* msg_norm_index, uint8_t* label_all, REAL* gap_min,
                         REAL* gap_norm, REAL* gap_label) {
  int64_t N = mpo_plane(g), P = mpo_pixels(g);
  REAL* U = (REAL*)malloc(sizeof(REAL) * N);
  for (int it = 0; it < n_iter; ++it) {
    for (int d = 0; d < g->n_dir; ++d) {
      int64_t io = ((int64_t)it * g->n_dir + d);
      FN(update_unary)(g, d, rho, unary, msg, U);
      FN(sweep)(g, d, rho, U, context, edge_weights + (int64_t)d * P, msg + (int64_t)d * N,
                msg_min_index ? msg_min_index + io * N : NULL,
                msg_norm_index ? msg_norm_index + io * P : NULL, gap_min ? gap_min + io * N : NULL,
                gap_norm ? gap_norm + io * P : NULL);
    }
    if (label_all) {
      FN(cost_aggregate)(g, enable_min_a_dir, 1, unary, msg, cost_final);
      FN(cal_label)(g, cost_final, label_all + (int64_t)it * P,
                    gap_label ? gap_label + (int64_t)it * P : NULL);
    }
  }
  FN(cost_aggregate)(g, enable_min_a_dir, 1, unary, msg, cost_final);
  free(U);
  return 0;
}

/* ---- ISGMR ForwardCUDA: ISGMR_forward.cu:433-665 (Jacobi over directions) --------------- */
/* msg_update must come in zero-filled as the reference's caller provides it                */
int FN(mpo_isgmr_forward)(const mpo_geom* g, int enable_sgm, REAL rho, int n_iter,
                          int enable_min_a_dir, const REAL* unary, const REAL* context,
                          const REAL* edge_weights, REAL* msg, REAL* msg_update, REAL* cost_final,
                          uint8_t* msg_min_index, uint8_t* msg_norm_index, uint8_t* label_all,
                          REAL* gap_min, REAL* gap_norm, REAL* gap_label) {
  int64_t N = mpo_plane(g), P = mpo_pixels(g);
  REAL* U = (REAL*)malloc(sizeof(REAL) * N);
  REAL factor = enable_sgm ? (REAL)g->n_dir : (REAL)1;
  for (int it = 0; it < n_iter; ++it) {
    for (int d = 0; d < g->n_dir; ++d) { /* every direction reads the OLD msg */
      int64_t io = ((int64_t)it * g->n_dir + d);
      FN(update_unary)(g, d, rho, unary, msg, U);
      FN(sweep)(g, d, rho, U, context, edge_weights + (int64_t)d * P, msg_update + (int64_t)d * N,
                msg_min_index ? msg_min_index + io * N : NULL,
                msg_norm_index ? msg_norm_index + io * P : NULL, gap_min ? gap_min + io * N : NULL,
                gap_norm ? gap_norm + io * P : NULL);
    }
    memcpy(msg, msg_update, sizeof(REAL) * N * g->n_dir); /* ISGMR_forward.cu:621-622 */
    if (label_all) {
      FN(cost_aggregate)(g, enable_min_a_dir, factor, unary, msg_update, cost_final);
      FN(cal_label)(g, cost_final, label_all + (int64_t)it * P,
                    gap_label ? gap_label + (int64_t)it * P : NULL);
    }
  }
  FN(cost_aggregate)(g, enable_min_a_dir, factor, unary, msg_update, cost_final);
  free(U);
  return 0;
}

/* ---- scan-back kernels: TRWP_backward.cu:49-275 (ISGMR_backward.cu:62-288 identical) ---- */
/* steps negated (common.cpp:89-92); front = current + negated step                          */
/* same_label: the hard kernels of the TRWP_hard_soft build, which add to dcontext without    */
/* the `current_d != front_d` guard (TRWP_hard_soft/TRWP_backward.cu:110,194,264)             */
static void FN(sweep_back)(const mpo_geom* g, int dir, REAL rho, const REAL* context,
                           const REAL* w_dir, const uint8_t* idx_min, const uint8_t* idx_norm,
                           REAL* dmsg_dir, REAL* dU, REAL* dcontext, REAL* dedge_dir,
                           int same_label) {
  int L = g->L, H = g->H, W = g->W;
  int hs, ws;
  mpo_dir_step(dir, &hs, &ws);
  hs = -hs;
  ws = -ws;
  int n_trees = mpo_n_trees(dir, H, W);
  REAL* gv = (REAL*)malloc(sizeof(REAL) * L);
  for (int bv = 0; bv < g->B; ++bv) {
    int64_t pix_base = (int64_t)bv * H * W;
    for (int tree = 0; tree < n_trees; ++tree) {
      int h0, w0, n_roll;
      mpo_tree_start(dir, hs, ws, H, W, tree, &h0, &w0, &n_roll);
      for (int i = 0; i <= n_roll; ++i) {
        int ch = h0 + i * hs, cw = w0 + i * ws;
        int fh = ch + hs, fw = cw + ws;
        if (ch < 0 || ch >= H || cw < 0 || cw >= W || fh < 0 || fh >= H || fw < 0 || fw >= W)
          continue;
        int64_t pc = pix_base + (int64_t)ch * W + cw;
        int64_t pf = pix_base + (int64_t)fh * W + fw;
        for (int l = 0; l < L; ++l) gv[l] = dmsg_dir[pc * L + l];
        /* MsgNormNaiveBack: commonCUDA.cuh:131-145 */
        REAL s = 0;
        for (int l = 0; l < L; ++l) s += gv[l];
        gv[idx_norm[pc]] += -s;
        for (int cd = 0; cd < L; ++cd) {
          int fd = idx_min[pc * L + cd];
          REAL v = gv[cd];
          int64_t co = FN(ctx_offset)(L, g->ctx2d, cd, fd);
          dU[pf * L + fd] += v;
          dmsg_dir[pf * L + fd] += rho * v;
          dedge_dir[pc] += context[co] * v;
          if (same_label || cd != fd) dcontext[co] += w_dir[pc] * v;
        }
      }
    }
  }
  free(gv);
}

/* ---- UpdateUnaryKernelBack: TRWP_backward.cu:26-47 --------------------------------------- */
static void FN(update_unary_back)(const mpo_geom* g, int dir, REAL rho, const REAL* dU,
                                  REAL* dunary, REAL* dmsg) {
  int64_t N = mpo_plane(g);
  int inv = dir ^ 1;
  for (int64_t i = 0; i < N; ++i) {
    REAL v = dU[i], vr = rho * v;
    for (int k = 0; k < g->n_dir; ++k) dmsg[(int64_t)k * N + i] += vr;
    dunary[i] += vr;
    dmsg[(int64_t)dir * N + i] += -vr;
    dmsg[(int64_t)inv * N + i] += -v;
  }
}

/* ---- TRWP BackwardCUDA: TRWP_backward.cu:277-433 ------------------------------------------ */
/* dcontext: (L,L) or (L,), dedge: (n_dir,B,H,W); both accumulate into the caller's values.    */
int FN(mpo_trwp_backward)(const mpo_geom* g, REAL rho, int n_iter, const REAL* context,
                          const REAL* edge_weights, const REAL* dcost_final,
                          const uint8_t* msg_min_index, const uint8_t* msg_norm_index,
                          REAL* dunary, REAL* dcontext, REAL* dedge_weights, int same_label) {
  int64_t N = mpo_plane(g), P = mpo_pixels(g);
  REAL* dmsg = (REAL*)malloc(sizeof(REAL) * N * g->n_dir);
  REAL* dU = (REAL*)calloc(N, sizeof(REAL));
  /* CostAggregateKernelBack: TRWP_backward.cu:8-24 */
  for (int64_t i = 0; i < N; ++i) {
    dunary[i] = dcost_final[i];
    for (int k = 0; k < g->n_dir; ++k) dmsg[(int64_t)k * N + i] = dcost_final[i];
  }
  for (int it = n_iter - 1; it >= 0; --it) {
    for (int d = g->n_dir - 1; d >= 0; --d) {
      int64_t io = ((int64_t)it * g->n_dir + d);
      FN(sweep_back)(g, d, rho, context, edge_weights + (int64_t)d * P, msg_min_index + io * N,
                     msg_norm_index + io * P, dmsg + (int64_t)d * N, dU, dcontext,
                     dedge_weights + (int64_t)d * P, same_label);
      FN(update_unary_back)(g, d, rho, dU, dunary, dmsg);
      memset(dU, 0, sizeof(REAL) * N);                    /* :421 */
      memset(dmsg + (int64_t)d * N, 0, sizeof(REAL) * N); /* :422 */
    }
  }
  free(dmsg);
  free(dU);
  return 0;
}

/* ---- ISGMR BackwardCUDA: ISGMR_backward.cu:290-493 ----------------------------------------- */
int FN(mpo_isgmr_backward)(const mpo_geom* g, int enable_sgm, REAL rho, int n_iter,
                           const REAL* context, const REAL* edge_weights, const REAL* dcost_final,
                           const uint8_t* msg_min_index, const uint8_t* msg_norm_index,
                           REAL* dunary, REAL* dcontext, REAL* dedge_weights) {
  int64_t N = mpo_plane(g), P = mpo_pixels(g);
  REAL* dmsg = (REAL*)malloc(sizeof(REAL) * N * g->n_dir);
  REAL* dmsg_update = (REAL*)malloc(sizeof(REAL) * N * g->n_dir);
  REAL* dU = (REAL*)calloc(N, sizeof(REAL));
  REAL factor = enable_sgm ? (REAL)g->n_dir : (REAL)1;
  /* CostAggregateKernelBack: ISGMR_backward.cu:18-37 */
  for (int64_t i = 0; i < N; ++i) {
    dunary[i] = factor * dcost_final[i];
    for (int k = 0; k < g->n_dir; ++k) dmsg_update[(int64_t)k * N + i] = dcost_final[i];
  }
  for (int it = n_iter - 1; it >= 0; --it) {
    memset(dmsg, 0, sizeof(REAL) * N * g->n_dir); /* :359 */
    for (int d = g->n_dir - 1; d >= 0; --d) {      /* diagonal, vertical, horizontal groups: d descending */
      int64_t io = ((int64_t)it * g->n_dir + d);
      FN(sweep_back)(g, d, rho, context, edge_weights + (int64_t)d * P, msg_min_index + io * N,
                     msg_norm_index + io * P, dmsg_update + (int64_t)d * N, dU, dcontext,
                     dedge_weights + (int64_t)d * P, 0);
      FN(update_unary_back)(g, d, rho, dU, dunary, dmsg);
      memset(dU, 0, sizeof(REAL) * N);
      memset(dmsg_update + (int64_t)d * N, 0, sizeof(REAL) * N);
    }
    /* SumMsgKernel + memcpy: :482-483 */
    for (int64_t i = 0; i < N * g->n_dir; ++i) dmsg[i] += dmsg_update[i];
    memcpy(dmsg_update, dmsg, sizeof(REAL) * N * g->n_dir);
  }
  free(dmsg);
  free(dmsg_update);
  free(dU);
  return 0;
}

/* =========================================================================================== */
/* Soft-weighted TRWP (MPLayers/TRWP_hard_soft): the min over front labels is replaced by the     */
/* expectation of the dual under softmin weights.                                                 */
/* =========================================================================================== */

/* offset of (cd, fd) inside a pixel's (L, L) block of msg_edge_label: even directions store      */
/* [fd][cd], odd ones [cd][fd] (is_pass_l2r = dir % 2 == 0, common.cpp:20;                        */
/* TRWP_forward_soft.cu:64)                                                                        */
static inline int64_t FN(soft_loc)(int L, int dir, int cd, int fd) {
  return (dir % 2 == 0) ? (int64_t)fd * L + cd : (int64_t)cd * L + fd;
}

/* softmin statistics of one row dual[0..L-1] (front labels): TRWP_forward_soft.cu:74-97.         */
/* prob may be NULL.  Returns the soft message sum_fd prob*dual.                                  */
static REAL FN(soft_row)(int L, const REAL* dual, REAL* prob) {
  REAL mn = dual[0];
  for (int fd = 1; fd < L; ++fd)
    if (dual[fd] < mn) mn = dual[fd];
  REAL s = 0;
  for (int fd = 0; fd < L; ++fd) s += (REAL)exp((double)(-dual[fd] + mn));
  REAL soft = 0;
  for (int fd = 0; fd < L; ++fd) {
    REAL e = (REAL)exp((double)(-dual[fd] + mn));
    if (prob) prob[fd] = e / s;
    soft += e * dual[fd] / s;
  }
  return soft;
}

/* one pixel of DynamicProgramming: TRWP_forward_soft.cu:9-117.  edge_label: the pixel's (L,L)     */
/* block or NULL.  Norm index: largest label on ties (TRWP_soft.cuh:104-108, torch >= 1).          */
static void FN(pixel_step_soft)(int L, int ctx2d, int dir, REAL rho, const REAL* Ufront,
                                const REAL* context, REAL w, REAL* prev, REAL* tmp, REAL* row,
                                REAL* m_out, REAL* edge_label, uint8_t* idx_norm) {
  for (int cd = 0; cd < L; ++cd) {
    for (int fd = 0; fd < L; ++fd) {
      REAL cv = context[FN(ctx_offset)(L, ctx2d, cd, fd)];
      row[fd] = Ufront[fd] + rho * prev[fd] + w * cv; /* :69 */
      if (edge_label) edge_label[FN(soft_loc)(L, dir, cd, fd)] = row[fd];
    }
    tmp[cd] = FN(soft_row)(L, row, NULL);
  }
  REAL nmin = tmp[0];
  int narg = 0;
  for (int cd = 1; cd < L; ++cd)
    if (tmp[cd] <= nmin) { /* equal: the larger index wins */
      nmin = tmp[cd];
      narg = cd;
    }
  for (int cd = 0; cd < L; ++cd) {
    prev[cd] = tmp[cd] - nmin;
    m_out[cd] = prev[cd];
  }
  if (idx_norm) *idx_norm = (uint8_t)narg;
}

/* Horizontal/DiagonalWide/DiagonalNarrow KernelSoft: TRWP_forward_soft.cu:183-376 (same chain     */
/* geometry as the hard kernels)                                                                   */
static void FN(sweep_soft)(const mpo_geom* g, int dir, REAL rho, const REAL* U, const REAL* context,
                           const REAL* w_dir, REAL* m_out, REAL* edge_label, uint8_t* idx_norm) {
  int L = g->L, H = g->H, W = g->W;
  int hs, ws;
  mpo_dir_step(dir, &hs, &ws);
  int n_trees = mpo_n_trees(dir, H, W);
  REAL* prev = (REAL*)malloc(sizeof(REAL) * L);
  REAL* tmp = (REAL*)malloc(sizeof(REAL) * L);
  REAL* row = (REAL*)malloc(sizeof(REAL) * L);
  for (int bv = 0; bv < g->B; ++bv) {
    int64_t pix_base = (int64_t)bv * H * W;
    for (int tree = 0; tree < n_trees; ++tree) {
      int h0, w0, n_roll;
      mpo_tree_start(dir, hs, ws, H, W, tree, &h0, &w0, &n_roll);
      for (int l = 0; l < L; ++l) prev[l] = 0;
      for (int i = 0; i <= n_roll; ++i) {
        int ch = h0 + i * hs, cw = w0 + i * ws;
        int fh = ch - hs, fw = cw - ws;
        if (ch < 0 || ch >= H || cw < 0 || cw >= W || fh < 0 || fh >= H || fw < 0 || fw >= W)
          continue;
        int64_t pc = pix_base + (int64_t)ch * W + cw;
        int64_t pf = pix_base + (int64_t)fh * W + fw;
        FN(pixel_step_soft)(L, g->ctx2d, dir, rho, U + pf * L, context, w_dir[pc], prev, tmp, row,
                            m_out + pc * L, edge_label ? edge_label + pc * L * L : NULL,
                            idx_norm ? idx_norm + pc : NULL);
      }
    }
  }
  free(prev);
  free(tmp);
  free(row);
}

/* ForwardCUDASoft: TRWP_forward_soft.cu:378-559.  msg_edge_label (n_iter,n_dir,B,H,W,L,L) and      */
/* msg_norm_index (n_iter,n_dir,B,H,W) may both be NULL (inference).                               */
int FN(mpo_trwp_soft_forward)(const mpo_geom* g, REAL rho, int n_iter, const REAL* unary,
                              const REAL* context, const REAL* edge_weights, REAL* msg,
                              REAL* cost_final, REAL* msg_edge_label, uint8_t* msg_norm_index,
                              uint8_t* label_all, REAL* gap_label) {
  int64_t N = mpo_plane(g), P = mpo_pixels(g);
  REAL* U = (REAL*)malloc(sizeof(REAL) * N);
  for (int it = 0; it < n_iter; ++it) {
    for (int d = 0; d < g->n_dir; ++d) {
      int64_t io = ((int64_t)it * g->n_dir + d);
      FN(update_unary)(g, d, rho, unary, msg, U); /* UpdateUnaryKernelSoft :161-181, same formula */
      FN(sweep_soft)(g, d, rho, U, context, edge_weights + (int64_t)d * P, msg + (int64_t)d * N,
                     msg_edge_label ? msg_edge_label + io * N * g->L : NULL,
                     msg_norm_index ? msg_norm_index + io * P : NULL);
    }
    if (label_all) {
      FN(cost_aggregate)(g, 0, 1, unary, msg, cost_final); /* CostAggregateKernelSoft :142-159 */
      FN(cal_label)(g, cost_final, label_all + (int64_t)it * P, /* CalLabelKernelSoft :119-140 */
                    gap_label ? gap_label + (int64_t)it * P : NULL);
    }
  }
  FN(cost_aggregate)(g, 0, 1, unary, msg, cost_final);
  free(U);
  return 0;
}

/* DynamicProgrammingBack over one direction: TRWP_backward_soft.cu:9-129, 170-420                  */
static void FN(sweep_back_soft)(const mpo_geom* g, int dir, REAL rho, const REAL* context,
                                const REAL* w_dir, const REAL* edge_label, const uint8_t* idx_norm,
                                REAL* dmsg_dir, REAL* dU, REAL* dcontext, REAL* dedge_dir) {
  int L = g->L, H = g->H, W = g->W;
  int hs, ws;
  mpo_dir_step(dir, &hs, &ws);
  hs = -hs;
  ws = -ws;
  int n_trees = mpo_n_trees(dir, H, W);
  REAL* gv = (REAL*)malloc(sizeof(REAL) * L);
  REAL* row = (REAL*)malloc(sizeof(REAL) * L);
  REAL* prob = (REAL*)malloc(sizeof(REAL) * L);
  for (int bv = 0; bv < g->B; ++bv) {
    int64_t pix_base = (int64_t)bv * H * W;
    for (int tree = 0; tree < n_trees; ++tree) {
      int h0, w0, n_roll;
      mpo_tree_start(dir, hs, ws, H, W, tree, &h0, &w0, &n_roll);
      for (int i = 0; i <= n_roll; ++i) {
        int ch = h0 + i * hs, cw = w0 + i * ws;
        int fh = ch + hs, fw = cw + ws;
        if (ch < 0 || ch >= H || cw < 0 || cw >= W || fh < 0 || fh >= H || fw < 0 || fw >= W)
          continue;
        int64_t pc = pix_base + (int64_t)ch * W + cw;
        int64_t pf = pix_base + (int64_t)fh * W + fw;
        for (int l = 0; l < L; ++l) gv[l] = dmsg_dir[pc * L + l];
        REAL s = 0; /* back norm :52-63 */
        for (int l = 0; l < L; ++l) s += gv[l];
        gv[idx_norm[pc]] -= s;
        for (int cd = 0; cd < L; ++cd) {
          for (int fd = 0; fd < L; ++fd) row[fd] = edge_label[pc * L * L + FN(soft_loc)(L, dir, cd, fd)];
          REAL soft = FN(soft_row)(L, row, prob); /* :83-105 */
          for (int fd = 0; fd < L; ++fd) {
            REAL dd = gv[cd] * prob[fd] * (1 - row[fd] + soft); /* :110-113 */
            int64_t co = FN(ctx_offset)(L, g->ctx2d, cd, fd);
            dU[pf * L + fd] += dd;
            dmsg_dir[pf * L + fd] += rho * dd;
            dedge_dir[pc] += context[co] * dd;
            dcontext[co] += w_dir[pc] * dd; /* every pair, the diagonal included :126 */
          }
        }
      }
    }
  }
  free(gv);
  free(row);
  free(prob);
}

/* BackwardCUDASoft: TRWP_backward_soft.cu:422-548 */
int FN(mpo_trwp_soft_backward)(const mpo_geom* g, REAL rho, int n_iter, const REAL* context,
                               const REAL* edge_weights, const REAL* dcost_final,
                               const REAL* msg_edge_label, const uint8_t* msg_norm_index,
                               REAL* dunary, REAL* dcontext, REAL* dedge_weights) {
  int64_t N = mpo_plane(g), P = mpo_pixels(g);
  REAL* dmsg = (REAL*)malloc(sizeof(REAL) * N * g->n_dir);
  REAL* dU = (REAL*)calloc(N, sizeof(REAL));
  for (int64_t i = 0; i < N; ++i) { /* CostAggregateKernelSoftBack :131-147 */
    dunary[i] = dcost_final[i];
    for (int k = 0; k < g->n_dir; ++k) dmsg[(int64_t)k * N + i] = dcost_final[i];
  }
  for (int it = n_iter - 1; it >= 0; --it) {
    for (int d = g->n_dir - 1; d >= 0; --d) {
      int64_t io = ((int64_t)it * g->n_dir + d);
      FN(sweep_back_soft)(g, d, rho, context, edge_weights + (int64_t)d * P,
                          msg_edge_label + io * N * g->L, msg_norm_index + io * P,
                          dmsg + (int64_t)d * N, dU, dcontext, dedge_weights + (int64_t)d * P);
      FN(update_unary_back)(g, d, rho, dU, dunary, dmsg); /* UpdateUnaryKernelSoftBack :149-168 */
      memset(dU, 0, sizeof(REAL) * N);                    /* :535 */
      memset(dmsg + (int64_t)d * N, 0, sizeof(REAL) * N); /* :536 */
    }
  }
  free(dmsg);
  free(dU);
  return 0;
}
