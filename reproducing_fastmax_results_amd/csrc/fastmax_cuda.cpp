// Torch binding "fastmax_cuda": the reference extension's two entry points
// (reference fastmax_cuda.cpp:17-37) on top of the C ABI of libfastmax_hip.so,
// plus stride-aware variants that avoid the wrapper's layout copies.
//
// Host-only C++: tensors are unpacked to pointers and strides, scratch comes
// from torch's caching allocator, work is enqueued on torch's current HIP
// stream, and nothing synchronises.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include <cmath>
#include <tuple>
#include <vector>

#include "fastmax_hip.h"

namespace {

#define FM_CHECK_CUDA(x) TORCH_CHECK((x).device().is_cuda(), #x " must be a CUDA tensor")
#define FM_CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define FM_CHECK_INPUT(x) \
  FM_CHECK_CUDA(x);       \
  FM_CHECK_CONTIGUOUS(x)

void check_status(int st, const char* what) {
  TORCH_CHECK(st == FASTMAX_OK, what, ": ", fastmax_status_string(st), " (status ", st, ")");
}

int dtype_code(const torch::Tensor& t) {
  if (t.scalar_type() == torch::kFloat32) return FASTMAX_F32;
  if (t.scalar_type() == torch::kBFloat16) return FASTMAX_BF16;
  TORCH_CHECK(false, "fastmax: tensors must be float32 or bfloat16, got ", t.scalar_type());
  return -1;
}

void* stream_of(const torch::Tensor& t) {
  return static_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

torch::Tensor workspace(size_t bytes, const torch::Tensor& like) {
  return torch::empty({static_cast<int64_t>(bytes)}, like.options().dtype(torch::kUInt8));
}

// (n, bh, d) contiguous tensor seen as (bh, n, d)
FastmaxStrides legacy_strides(int64_t bh, int64_t width) { return FastmaxStrides{width, bh * width}; }

void scale_or_normalize(torch::Tensor& x, int64_t bh, int64_t n, int64_t d, bool max_norm, float scale) {
  FastmaxNormDesc nd{};
  nd.bh = static_cast<int32_t>(bh); nd.n = static_cast<int32_t>(n); nd.d = static_cast<int32_t>(d);
  nd.dtype = dtype_code(x); nd.centre = 0; nd.max_norm = max_norm ? 1 : 0; nd.scale = scale;
  nd.sx = legacy_strides(bh, d); nd.sy = nd.sx;
  torch::Tensor stats = torch::empty({bh * (d + 2)}, x.options().dtype(torch::kFloat32));
  check_status(fastmax_normalize(&nd, x.data_ptr(), x.data_ptr(), stats.data_ptr<float>(), stream_of(x)),
               "fastmax_normalize");
}

FastmaxDesc legacy_desc(const torch::Tensor& q, const torch::Tensor& k, bool mask, float a0, float a1, float a2,
                        int64_t p) {
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3, "q, k, v must be (n, b*h, d)");
  FastmaxDesc d{};
  d.nq = static_cast<int32_t>(q.size(0)); d.nk = static_cast<int32_t>(k.size(0));
  d.bh = static_cast<int32_t>(q.size(1)); d.d = static_cast<int32_t>(q.size(2));
  d.dtype = dtype_code(q);
  d.mask = mask ? 1 : 0; d.p = static_cast<int32_t>(p);
  d.a0 = a0; d.a1 = a1; d.a2 = a2; d.inv_tau = 1.0f;    // the temperature is already in k
  d.chunk = 0; d.flags = 0;
  d.sq = legacy_strides(d.bh, d.d); d.sk = d.sq; d.sv = d.sq;
  d.sdo = d.sq; d.sdq = d.sq; d.sdk = d.sq; d.sdv = d.sq;
  return d;
}

// ---------------------------------------------------------------------------------
// forwardpass: same signature and result as the reference (fastmax_cuda.cpp:17).
// q (nq, bh, d), k, v (nk, bh, d); returns (nq, bh, d+1) float32 with the
// denominator in the last column.  Like the reference it leaves k divided by the
// temperature (and q, k normalised when `normalize`) IN PLACE, because the
// reference's autograd wrapper saves those tensors and hands them to backwardpass
// (transformer/model.py:29-37, fastmax_cuda_forward.cu:288,335).  drop_noise,
// rpe_matrix and dropout are accepted and ignored, as in the reference
// (fastmax_cuda_forward.cu:289 commented out, :443 scale 0).
// `normalize` implements lim * x / max_n ||x_n||_2 (transformer/model.py:97-102).
// ---------------------------------------------------------------------------------
torch::Tensor forwardpass(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor drop_noise,
                          torch::Tensor rpe_matrix, bool mask, double dropout, bool normalize, double temperature,
                          double a0, double a1, double a2, double lim, int64_t p) {
  FM_CHECK_INPUT(q);
  FM_CHECK_INPUT(k);
  FM_CHECK_INPUT(v);
  (void)drop_noise; (void)rpe_matrix; (void)dropout;
  FastmaxDesc d = legacy_desc(q, k, mask, float(a0), float(a1), float(a2), p);
  TORCH_CHECK(v.dim() == 3 && v.sizes() == k.sizes(), "v must have k's shape");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "q, k, v must share one dtype");
  scale_or_normalize(k, d.bh, d.nk, d.d, false, float(1.0 / temperature));
  if (normalize) {
    scale_or_normalize(q, d.bh, d.nq, d.d, true, float(lim));
    scale_or_normalize(k, d.bh, d.nk, d.d, true, float(lim));
  }
  size_t fwd = 0, bwd = 0;
  check_status(fastmax_workspace_bytes(&d, &fwd, &bwd), "fastmax_workspace_bytes");
  torch::Tensor ws = workspace(fwd, q);
  torch::Tensor out = torch::empty({d.nq, d.bh, d.d + 1}, q.options().dtype(torch::kFloat32));
  if (d.dtype == FASTMAX_F32) {
    d.so = legacy_strides(d.bh, d.d + 1);
    d.sg = d.so;
    float* op = out.data_ptr<float>();
    check_status(fastmax_forward(&d, q.data_ptr(), k.data_ptr(), v.data_ptr(), op, op + d.d, ws.data_ptr(), fwd,
                                 stream_of(q)), "fastmax_forward");
  } else {
    torch::Tensor o = torch::empty({d.nq, d.bh, d.d}, q.options());
    torch::Tensor g = torch::empty({d.nq, d.bh}, q.options().dtype(torch::kFloat32));
    d.so = legacy_strides(d.bh, d.d);
    d.sg = FastmaxStrides{1, d.bh};
    check_status(fastmax_forward(&d, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), g.data_ptr<float>(),
                                 ws.data_ptr(), fwd, stream_of(q)), "fastmax_forward");
    out.narrow(2, 0, d.d).copy_(o);
    out.select(2, d.d).copy_(g);
  }
  return out;
}

// backwardpass: same signature and result as the reference (fastmax_cuda.cpp:26).
// q, k: the tensors as left by forwardpass; o: its (nq, bh, d+1) result.
// grad_output is not modified.
std::vector<torch::Tensor> backwardpass(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor o,
                                        torch::Tensor grad_output, bool mask, double a0, double a1, double a2,
                                        int64_t p) {
  FM_CHECK_INPUT(q);
  FM_CHECK_INPUT(k);
  FM_CHECK_INPUT(v);
  FastmaxDesc d = legacy_desc(q, k, mask, float(a0), float(a1), float(a2), p);
  TORCH_CHECK(o.dim() == 3 && o.size(0) == d.nq && o.size(1) == d.bh && o.size(2) == d.d + 1 &&
                  o.scalar_type() == torch::kFloat32 && o.is_contiguous(),
              "o must be the contiguous float32 (nq, bh, d+1) result of forwardpass");
  torch::Tensor go = grad_output.contiguous();
  TORCH_CHECK(go.sizes() == q.sizes() && go.scalar_type() == q.scalar_type(), "grad_output must match q");
  torch::Tensor gq = torch::empty_like(q), gk = torch::empty_like(k), gv = torch::empty_like(v);
  torch::Tensor ov = o;
  const float* gp = o.data_ptr<float>() + d.d;
  d.sg = legacy_strides(d.bh, d.d + 1);
  if (d.dtype == FASTMAX_F32) {
    d.so = legacy_strides(d.bh, d.d + 1);
  } else {
    ov = o.narrow(2, 0, d.d).to(q.scalar_type()).contiguous();
    d.so = legacy_strides(d.bh, d.d);
  }
  size_t fwd = 0, bwd = 0;
  check_status(fastmax_workspace_bytes(&d, &fwd, &bwd), "fastmax_workspace_bytes");
  torch::Tensor ws = workspace(bwd, q);
  check_status(fastmax_backward(&d, q.data_ptr(), k.data_ptr(), v.data_ptr(), ov.data_ptr(), gp, go.data_ptr(),
                                gq.data_ptr(), gk.data_ptr(), gv.data_ptr(), ws.data_ptr(), bwd, stream_of(q)),
               "fastmax_backward");
  return {gq, gk, gv};
}

// ---------------------------------------------------------------------------------
// Stride-aware entry points: any (bh, n, d) view (3-D) or (b, h, n, d) tensor whose
// feature axis is contiguous and whose batch and head axes collapse to one stride.
// ---------------------------------------------------------------------------------
torch::Tensor as_bhnd(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 3 || t.dim() == 4, name, " must be (bh, n, d) or (b, h, n, d)");
  torch::Tensor x = t;
  if (x.size(-1) > 1 && x.stride(-1) != 1) x = x.contiguous();
  if (x.dim() == 4) {
    if (x.size(0) > 1 && x.size(1) > 1 && x.stride(0) != x.size(1) * x.stride(1)) x = x.contiguous();
    const int64_t sbh = x.size(1) > 1 ? x.stride(1) : x.stride(0);
    x = x.as_strided({x.size(0) * x.size(1), x.size(2), x.size(3)}, {sbh, x.stride(2), x.stride(3)}, x.storage_offset());
  }
  return x;
}

FastmaxStrides strides_of(const torch::Tensor& t) { return FastmaxStrides{t.stride(0), t.stride(1)}; }

FastmaxDesc ex_desc(const torch::Tensor& q, const torch::Tensor& k, const torch::Tensor& v, bool mask, double inv_tau,
                    double a0, double a1, double a2, int64_t p, int64_t chunk, int64_t flags) {
  FM_CHECK_CUDA(q); FM_CHECK_CUDA(k); FM_CHECK_CUDA(v);
  TORCH_CHECK(k.size(0) == q.size(0) && v.size(0) == q.size(0) && k.size(2) == q.size(2) && v.size(2) == q.size(2) &&
                  v.size(1) == k.size(1), "q, k, v must be (bh, nq, d), (bh, nk, d), (bh, nk, d)");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "q, k, v must share one dtype");
  FastmaxDesc d{};
  d.bh = static_cast<int32_t>(q.size(0)); d.nq = static_cast<int32_t>(q.size(1)); d.nk = static_cast<int32_t>(k.size(1));
  d.d = static_cast<int32_t>(q.size(2)); d.dtype = dtype_code(q);
  d.mask = mask ? 1 : 0; d.p = static_cast<int32_t>(p);
  d.a0 = float(a0); d.a1 = float(a1); d.a2 = float(a2); d.inv_tau = float(inv_tau);
  d.chunk = static_cast<int32_t>(chunk); d.flags = static_cast<int32_t>(flags);
  d.sq = strides_of(q); d.sk = strides_of(k); d.sv = strides_of(v);
  return d;
}

std::vector<torch::Tensor> forward_any(torch::Tensor q_, torch::Tensor k_, torch::Tensor v_, bool mask, double inv_tau,
                                       double a0, double a1, double a2, int64_t p, int64_t chunk, int64_t flags) {
  torch::Tensor q = as_bhnd(q_, "q"), k = as_bhnd(k_, "k"), v = as_bhnd(v_, "v");
  FastmaxDesc d = ex_desc(q, k, v, mask, inv_tau, a0, a1, a2, p, chunk, flags);
  torch::Tensor o = torch::empty({d.bh, d.nq, d.d}, q.options());
  torch::Tensor g = torch::empty({d.bh, d.nq}, q.options().dtype(torch::kFloat32));
  d.so = strides_of(o);
  d.sg = FastmaxStrides{g.stride(0), g.stride(1)};
  size_t fwd = 0, bwd = 0;
  check_status(fastmax_workspace_bytes(&d, &fwd, &bwd), "fastmax_workspace_bytes");
  torch::Tensor ws = workspace(fwd, q);
  check_status(fastmax_forward(&d, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), g.data_ptr<float>(),
                               ws.data_ptr(), fwd, stream_of(q)), "fastmax_forward");
  if (q_.dim() == 4) return {o.view({q_.size(0), q_.size(1), d.nq, d.d}), g.view({q_.size(0), q_.size(1), d.nq}), ws};
  return {o, g, ws};
}

std::tuple<torch::Tensor, torch::Tensor> forward_ex(torch::Tensor q, torch::Tensor k, torch::Tensor v, bool mask,
                                                    double inv_tau, double a0, double a1, double a2, int64_t p,
                                                    int64_t chunk, int64_t flags) {
  std::vector<torch::Tensor> r = forward_any(q, k, v, mask, inv_tau, a0, a1, a2, p, chunk,
                                             flags & ~int64_t(FASTMAX_FLAG_SAVE_FOR_BACKWARD));
  return {r[0], r[1]};
}

// Forward that keeps its workspace (key-side copies and prefix states) for backward_saved.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> forward_save(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                                                                   bool mask, double inv_tau, double a0, double a1,
                                                                   double a2, int64_t p, int64_t chunk, int64_t flags) {
  std::vector<torch::Tensor> r = forward_any(q, k, v, mask, inv_tau, a0, a1, a2, p, chunk,
                                             flags | FASTMAX_FLAG_SAVE_FOR_BACKWARD);
  return {r[0], r[1], r[2]};
}

std::vector<torch::Tensor> backward_any(torch::Tensor q_, torch::Tensor k_, torch::Tensor v_, torch::Tensor o_,
                                        torch::Tensor g_, torch::Tensor go_, const torch::Tensor* saved, bool mask,
                                        double inv_tau, double a0, double a1, double a2, int64_t p, int64_t chunk,
                                        int64_t flags) {
  torch::Tensor q = as_bhnd(q_, "q"), k = as_bhnd(k_, "k"), v = as_bhnd(v_, "v");
  torch::Tensor o = as_bhnd(o_, "o"), go = as_bhnd(go_, "grad_output");
  FastmaxDesc d = ex_desc(q, k, v, mask, inv_tau, a0, a1, a2, p, chunk, flags);
  TORCH_CHECK(o.scalar_type() == q.scalar_type() && go.scalar_type() == q.scalar_type(), "o and grad_output must match q");
  TORCH_CHECK(g_.scalar_type() == torch::kFloat32 && g_.numel() == int64_t(d.bh) * d.nq, "g must be float32 (bh, nq)");
  torch::Tensor g = g_.contiguous().view({d.bh, d.nq});
  torch::Tensor dq = torch::empty({d.bh, d.nq, d.d}, q.options());
  torch::Tensor dk = torch::empty({d.bh, d.nk, d.d}, q.options());
  torch::Tensor dv = torch::empty({d.bh, d.nk, d.d}, q.options());
  d.so = strides_of(o); d.sdo = strides_of(go);
  d.sg = FastmaxStrides{g.stride(0), g.stride(1)};
  d.sdq = strides_of(dq); d.sdk = strides_of(dk); d.sdv = strides_of(dv);
  size_t fwd = 0, bwd = 0;
  check_status(fastmax_workspace_bytes(&d, &fwd, &bwd), "fastmax_workspace_bytes");
  torch::Tensor ws = workspace(bwd, q);
  if (saved) {
    TORCH_CHECK(saved->is_cuda() && saved->scalar_type() == torch::kUInt8 && saved->is_contiguous(),
                "saved workspace must be the uint8 tensor returned by forward_save");
    check_status(fastmax_backward_saved(&d, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), g.data_ptr<float>(),
                                        go.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), saved->data_ptr(),
                                        size_t(saved->numel()), ws.data_ptr(), bwd, stream_of(q)),
                 "fastmax_backward_saved");
  } else {
    check_status(fastmax_backward(&d, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), g.data_ptr<float>(),
                                  go.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), bwd,
                                  stream_of(q)), "fastmax_backward");
  }
  if (q_.dim() == 4) {
    const int64_t b = q_.size(0), h = q_.size(1);
    return {dq.view({b, h, d.nq, d.d}), dk.view({b, h, d.nk, d.d}), dv.view({b, h, d.nk, d.d})};
  }
  return {dq, dk, dv};
}

std::vector<torch::Tensor> backward_ex(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor o,
                                       torch::Tensor g, torch::Tensor go, bool mask, double inv_tau, double a0,
                                       double a1, double a2, int64_t p, int64_t chunk, int64_t flags) {
  return backward_any(q, k, v, o, g, go, nullptr, mask, inv_tau, a0, a1, a2, p, chunk,
                      flags & ~int64_t(FASTMAX_FLAG_SAVE_FOR_BACKWARD));
}

// Backward on the workspace forward_save returned for the same q, k, v and parameters.
std::vector<torch::Tensor> backward_saved(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor o,
                                          torch::Tensor g, torch::Tensor go, torch::Tensor saved, bool mask,
                                          double inv_tau, double a0, double a1, double a2, int64_t p, int64_t chunk,
                                          int64_t flags) {
  return backward_any(q, k, v, o, g, go, &saved, mask, inv_tau, a0, a1, a2, p, chunk,
                      flags | FASTMAX_FLAG_SAVE_FOR_BACKWARD);
}

// y = scale * (x - centre) / max_n ||x_n - centre||  (see fastmax_normalize in the C header)
torch::Tensor normalize(torch::Tensor x_, int64_t centre, bool max_norm, double scale) {
  torch::Tensor x = as_bhnd(x_, "x");
  FM_CHECK_CUDA(x);
  FastmaxNormDesc nd{};
  nd.bh = static_cast<int32_t>(x.size(0)); nd.n = static_cast<int32_t>(x.size(1)); nd.d = static_cast<int32_t>(x.size(2));
  nd.dtype = dtype_code(x); nd.centre = static_cast<int32_t>(centre); nd.max_norm = max_norm ? 1 : 0;
  nd.scale = float(scale);
  torch::Tensor y = torch::empty({nd.bh, nd.n, nd.d}, x.options());
  nd.sx = strides_of(x); nd.sy = strides_of(y);
  torch::Tensor stats = torch::empty({int64_t(nd.bh) * (nd.d + 2)}, x.options().dtype(torch::kFloat32));
  check_status(fastmax_normalize(&nd, x.data_ptr(), y.data_ptr(), stats.data_ptr<float>(), stream_of(x)),
               "fastmax_normalize");
  return x_.dim() == 4 ? y.view(x_.sizes()) : y;
}

}  // namespace

PYBIND11_MODULE(fastmax_cuda, m) {
  m.def("forwardpass", &forwardpass, "forwardpass");
  m.def("backwardpass", &backwardpass, "backwardpass");
  m.def("forward_ex", &forward_ex, "strided forward: returns (o, g)");
  m.def("backward_ex", &backward_ex, "strided backward: returns [dq, dk, dv]");
  m.def("forward_save", &forward_save, "strided forward keeping its workspace: returns (o, g, saved)");
  m.def("backward_saved", &backward_saved, "strided backward on a saved forward workspace: returns [dq, dk, dv]");
  m.def("normalize", &normalize, "fused normalisation pass");
  m.def("version", []() { return fastmax_version(); });
}
