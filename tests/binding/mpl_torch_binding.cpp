// pybind11 operator modules over the C ABI of libmplayers_hip.so: the binding a maintainer of the
// reference puts in place of the bodies of Forward / Backward in MPLayers/TRWP/TRWP.cpp:245-326
// and MPLayers/ISGMR/ISGMR.cpp:300-404.  Same module names (TRWP, ISGMR), same function names
// (forward, backward), same positional arguments, caller-allocated tensors filled in place, an empty
// index / label tensor switches that output off.  Host code only: compiled with g++ against the
// torch headers, no device code and no nvcc / hipcc step.
//
// Built twice by build_binding.py: -DMPL_BIND_TRWP -> module TRWP, -DMPL_BIND_ISGMR -> module ISGMR.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include "mplayers_amd.h"

namespace {

// CHECK_CONTIGUOUS of the reference (tools/cuda/cudaUtils.hpp:10) plus what the reference leaves
// unchecked and the C ABI relies on: device, dtype and size of every tensor
void check(const at::Tensor& t, const char* name, at::ScalarType dtype, int64_t numel,
           bool cuda = true) {
  TORCH_CHECK(t.is_cuda() == cuda, name, cuda ? " must be a GPU tensor like the rest of the call"
                                              : " must be a CPU tensor like the rest of the call");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(t.scalar_type() == dtype, name, " has the wrong dtype");
  TORCH_CHECK(t.numel() >= numel, name, " has ", t.numel(), " elements, ", numel, " needed");
}

// msg: (n_dir, batch, cv, h, w, n_disp), as ForwardCUDA reads it (TRWP_forward.cu:390-395)
mpl_shape shape_of(const at::Tensor& msg) {
  TORCH_CHECK(msg.dim() == 6, "msg must be (n_dir, batch, cv, h, w, n_disp)");
  mpl_shape s = {};
  s.n_dir = (int)msg.size(0);
  s.batch = (int)(msg.size(1) * msg.size(2));
  s.height = (int)msg.size(3);
  s.width = (int)msg.size(4);
  s.n_disp = (int)msg.size(5);
  s.ctx2d = (s.n_disp == 21) ? 1 : 0;  // the reference's segmentation switch (TRWP_forward.cu:101)
  return s;
}

// msg_min_index: (n_iter, n_dir, batch, cv, h, w, n_disp), as BackwardCUDA reads it
// (TRWP_backward.cu:288-294)
mpl_shape shape_of_index(const at::Tensor& idx, int* n_iter) {
  TORCH_CHECK(idx.dim() == 7, "msg_min_index must be (n_iter, n_dir, batch, cv, h, w, n_disp)");
  mpl_shape s = {};
  *n_iter = (int)idx.size(0);
  s.n_dir = (int)idx.size(1);
  s.batch = (int)(idx.size(2) * idx.size(3));
  s.height = (int)idx.size(4);
  s.width = (int)idx.size(5);
  s.n_disp = (int)idx.size(6);
  s.ctx2d = (s.n_disp == 21) ? 1 : 0;
  return s;
}

int64_t pixels(const mpl_shape& s) { return (int64_t)s.batch * s.height * s.width; }
int64_t context_numel(const mpl_shape& s) { return s.ctx2d ? s.n_disp * s.n_disp : s.n_disp; }
uint8_t* u8_or_null(const at::Tensor& t) { return t.numel() ? t.data_ptr<uint8_t>() : nullptr; }
float* f32_or_null(const at::Tensor& t) { return t.numel() ? t.data_ptr<float>() : nullptr; }

void check_forward(const mpl_shape& s, int n_iter, const at::Tensor& unary,
                   const at::Tensor& context, const at::Tensor& edge_weights, const at::Tensor& msg,
                   const at::Tensor& cost_final, const at::Tensor& msg_min_index,
                   const at::Tensor& msg_norm_index, const at::Tensor& unary_update,
                   const at::Tensor& label_all) {
  const int64_t P = pixels(s), N = P * s.n_disp;
  check(unary, "unary", at::kFloat, N);
  check(context, "context", at::kFloat, context_numel(s));
  check(edge_weights, "edge_weights", at::kFloat, s.n_dir * P);
  check(msg, "msg", at::kFloat, s.n_dir * N);
  check(cost_final, "cost_final", at::kFloat, N);
  check(unary_update, "unary_update", at::kFloat, N);
  if (msg_min_index.numel() > 0) {
    check(msg_min_index, "msg_min_index", at::kByte, (int64_t)n_iter * s.n_dir * N);
    check(msg_norm_index, "msg_norm_index", at::kByte, (int64_t)n_iter * s.n_dir * P);
  }
  if (label_all.numel() > 0) check(label_all, "label_all", at::kByte, (int64_t)n_iter * P);
}

void check_backward(const mpl_shape& s, int n_iter, const at::Tensor& context,
                    const at::Tensor& edge_weights, const at::Tensor& dcost_final,
                    const at::Tensor& msg_min_index, const at::Tensor& msg_norm_index,
                    const at::Tensor& dunary, const at::Tensor& dcontext,
                    const at::Tensor& dedge_weights) {
  const int64_t P = pixels(s), N = P * s.n_disp;
  check(context, "context", at::kFloat, context_numel(s));
  check(edge_weights, "edge_weights", at::kFloat, s.n_dir * P);
  check(dcost_final, "dcost_final", at::kFloat, N);
  check(msg_min_index, "msg_min_index", at::kByte, (int64_t)n_iter * s.n_dir * N);
  check(msg_norm_index, "msg_norm_index", at::kByte, (int64_t)n_iter * s.n_dir * P);
  check(dunary, "dunary", at::kFloat, N);
  check(dcontext, "dcontext", at::kFloat, context_numel(s));
  check(dedge_weights, "dedge_weights", at::kFloat, s.n_dir * P);
}

// Tensors that are not on the GPU: ForwardCPU of the reference (TRWP.cpp:172-243 reached from
// :275-282, ISGMR.cpp:190-298 from :330-339) through the library's CPU entry points.  That path
// reads one pairwise table per direction at context + d * n_disp^2 and ignores edge weights,
// indices and unary_update.
void check_forward_cpu(const mpl_shape& s, int n_iter, const at::Tensor& unary,
                       const at::Tensor& context, const at::Tensor& msg,
                       const at::Tensor& cost_final, const at::Tensor& label_all) {
  const int64_t P = pixels(s), N = P * s.n_disp;
  check(unary, "unary", at::kFloat, N, false);
  check(context, "context", at::kFloat,
        (int64_t)(s.n_dir - 1) * s.n_disp * s.n_disp + context_numel(s), false);
  check(msg, "msg", at::kFloat, s.n_dir * N, false);
  check(cost_final, "cost_final", at::kFloat, N, false);
  if (label_all.numel() > 0) check(label_all, "label_all", at::kByte, (int64_t)n_iter * P, false);
}

void* current_stream(const at::Tensor& t) {
  return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

#ifdef MPL_BIND_TRWP
// MPLayers/TRWP/TRWP.cpp:245-283
void Forward(const float rho, const int n_iter, const int enable_min_a_dir, const at::Tensor unary,
             const at::Tensor context, const at::Tensor edge_weights, at::Tensor msg,
             at::Tensor cost_final, at::Tensor msg_min_index, at::Tensor msg_norm_index,
             at::Tensor unary_update, at::Tensor label_all) {
  const mpl_shape s = shape_of(msg);
  if (!unary.is_cuda()) {
    check_forward_cpu(s, n_iter, unary, context, msg, cost_final, label_all);
    const int rc = mpl_trwp_forward_cpu(&s, rho, n_iter, unary.data_ptr<float>(),
                                        context.data_ptr<float>(), msg.data_ptr<float>(),
                                        cost_final.data_ptr<float>(), u8_or_null(label_all));
    TORCH_CHECK(rc == MPL_OK, "TRWP.forward: ", mpl_last_error());
    return;
  }
  check_forward(s, n_iter, unary, context, edge_weights, msg, cost_final, msg_min_index,
                msg_norm_index, unary_update, label_all);
  const c10::DeviceGuard guard(unary.device());
  const int rc = mpl_trwp_forward(&s, /*flags=*/0u, rho, n_iter, enable_min_a_dir,
                                  unary.data_ptr<float>(), context.data_ptr<float>(),
                                  edge_weights.data_ptr<float>(), msg.data_ptr<float>(),
                                  cost_final.data_ptr<float>(), u8_or_null(msg_min_index),
                                  u8_or_null(msg_norm_index), unary_update.data_ptr<float>(),
                                  u8_or_null(label_all), current_stream(unary));
  TORCH_CHECK(rc == MPL_OK, "TRWP.forward: ", mpl_last_error());
}

// MPLayers/TRWP/TRWP.cpp:285-318
void Backward(const float rho, const at::Tensor context, const at::Tensor edge_weights,
              const at::Tensor dcost_final, const at::Tensor msg_min_index,
              const at::Tensor msg_norm_index, at::Tensor dunary, at::Tensor dcontext,
              at::Tensor dedge_weights, at::Tensor dmsg, at::Tensor dunary_update) {
  // (the reference prints this and returns, TRWP.cpp:315-316)
  TORCH_CHECK(dcost_final.is_cuda(), "Does not support CPU backward.");
  int n_iter = 0;
  const mpl_shape s = shape_of_index(msg_min_index, &n_iter);
  check_backward(s, n_iter, context, edge_weights, dcost_final, msg_min_index, msg_norm_index,
                 dunary, dcontext, dedge_weights);
  check(dmsg, "dmsg", at::kFloat, s.n_dir * pixels(s) * s.n_disp);
  const c10::DeviceGuard guard(dcost_final.device());
  const int rc = mpl_trwp_backward(&s, /*flags=*/0u, rho, n_iter, context.data_ptr<float>(),
                                   edge_weights.data_ptr<float>(), dcost_final.data_ptr<float>(),
                                   msg_min_index.data_ptr<uint8_t>(),
                                   msg_norm_index.data_ptr<uint8_t>(), dunary.data_ptr<float>(),
                                   dcontext.data_ptr<float>(), dedge_weights.data_ptr<float>(),
                                   dmsg.data_ptr<float>(), f32_or_null(dunary_update),
                                   current_stream(dcost_final));
  TORCH_CHECK(rc == MPL_OK, "TRWP.backward: ", mpl_last_error());
}
#endif  // MPL_BIND_TRWP

#ifdef MPL_BIND_ISGMR
// MPLayers/ISGMR/ISGMR.cpp:300-342
void Forward(const int enable_sgm, const float rho, const int n_iter, const int enable_min_a_dir,
             const at::Tensor unary, const at::Tensor context, const at::Tensor edge_weights,
             at::Tensor msg, at::Tensor cost_final, at::Tensor msg_min_index,
             at::Tensor msg_norm_index, at::Tensor unary_update, at::Tensor msg_update,
             at::Tensor label_all) {
  const mpl_shape s = shape_of(msg);
  if (!unary.is_cuda()) {
    check_forward_cpu(s, n_iter, unary, context, msg, cost_final, label_all);
    check(msg_update, "msg_update", at::kFloat, s.n_dir * pixels(s) * s.n_disp, false);
    const int rc = mpl_isgmr_forward_cpu(&s, enable_sgm, rho, n_iter, unary.data_ptr<float>(),
                                         context.data_ptr<float>(), msg.data_ptr<float>(),
                                         cost_final.data_ptr<float>(), msg_update.data_ptr<float>(),
                                         u8_or_null(label_all));
    TORCH_CHECK(rc == MPL_OK, "ISGMR.forward: ", mpl_last_error());
    return;
  }
  check_forward(s, n_iter, unary, context, edge_weights, msg, cost_final, msg_min_index,
                msg_norm_index, unary_update, label_all);
  check(msg_update, "msg_update", at::kFloat, s.n_dir * pixels(s) * s.n_disp);
  const c10::DeviceGuard guard(unary.device());
  const int rc = mpl_isgmr_forward(&s, /*flags=*/0u, enable_sgm, rho, n_iter, enable_min_a_dir,
                                   unary.data_ptr<float>(), context.data_ptr<float>(),
                                   edge_weights.data_ptr<float>(), msg.data_ptr<float>(),
                                   cost_final.data_ptr<float>(), u8_or_null(msg_min_index),
                                   u8_or_null(msg_norm_index), unary_update.data_ptr<float>(),
                                   msg_update.data_ptr<float>(), u8_or_null(label_all),
                                   current_stream(unary));
  TORCH_CHECK(rc == MPL_OK, "ISGMR.forward: ", mpl_last_error());
}

// MPLayers/ISGMR/ISGMR.cpp:344-379
void Backward(const int enable_sgm, const float rho, const at::Tensor context,
              const at::Tensor edge_weights, const at::Tensor dcost_final,
              const at::Tensor msg_min_index, const at::Tensor msg_norm_index, at::Tensor dunary,
              at::Tensor dcontext, at::Tensor dedge_weights, at::Tensor dmsg,
              at::Tensor dunary_update, at::Tensor dmsg_update) {
  TORCH_CHECK(dcost_final.is_cuda(), "Does not support CPU backward.");  // ISGMR.cpp:377-378
  int n_iter = 0;
  const mpl_shape s = shape_of_index(msg_min_index, &n_iter);
  check_backward(s, n_iter, context, edge_weights, dcost_final, msg_min_index, msg_norm_index,
                 dunary, dcontext, dedge_weights);
  const int64_t planes = s.n_dir * pixels(s) * s.n_disp;
  check(dmsg, "dmsg", at::kFloat, planes);
  check(dmsg_update, "dmsg_update", at::kFloat, planes);
  const c10::DeviceGuard guard(dcost_final.device());
  const int rc = mpl_isgmr_backward(&s, /*flags=*/0u, enable_sgm, rho, n_iter,
                                    context.data_ptr<float>(), edge_weights.data_ptr<float>(),
                                    dcost_final.data_ptr<float>(),
                                    msg_min_index.data_ptr<uint8_t>(),
                                    msg_norm_index.data_ptr<uint8_t>(), dunary.data_ptr<float>(),
                                    dcontext.data_ptr<float>(), dedge_weights.data_ptr<float>(),
                                    dmsg.data_ptr<float>(), f32_or_null(dunary_update),
                                    dmsg_update.data_ptr<float>(), current_stream(dcost_final));
  TORCH_CHECK(rc == MPL_OK, "ISGMR.backward: ", mpl_last_error());
}
#endif  // MPL_BIND_ISGMR

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("forward", &Forward, "forward (HIP, libmplayers_hip.so)");
  m.def("backward", &Backward, "backward (HIP, libmplayers_hip.so)");
}
