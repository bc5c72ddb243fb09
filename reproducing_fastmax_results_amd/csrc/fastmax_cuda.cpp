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
  torch::Tensor stats = torch::empty({int64_t(fastmax_normalize_stats_bytes(&nd) / sizeof(float))},
                                     x.options().dtype(torch::kFloat32));
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
// Stride-aware entry points: any (bh, n, d) view (3-D) or (b, h, n, d) view (4-D) whose
// feature axis is contiguous is handed to the library as it lies in memory: a 3-D view with
// one stride for its first axis, a 4-D view with batch and head strides, so the transposed
// view of a (b, n, h*d) projection output needs no copy.
// ---------------------------------------------------------------------------------
struct View {
  torch::Tensor t;
  FastmaxStrides s;
  int64_t bh, n, d;
};

View view_of(const torch::Tensor& t_, const char* name) {
  TORCH_CHECK(t_.dim() == 3 || t_.dim() == 4, name, " must be (bh, n, d) or (b, h, n, d)");
  View w;
  w.t = (t_.size(-1) > 1 && t_.stride(-1) != 1) ? t_.contiguous() : t_;
  const torch::Tensor& x = w.t;
  if (x.dim() == 3) {
    w.s = FastmaxStrides{x.stride(0), x.stride(1), 0, 0, 0};
    w.bh = x.size(0); w.n = x.size(1); w.d = x.size(2);
  } else {
    // one head per batch: the batch stride is the stride of the whole batch*head axis (stride(1) of such
    // a view says nothing: for the projection layout (b, n, 1, d) transposed it is d)
    if (x.size(1) == 1) w.s = FastmaxStrides{x.stride(0), x.stride(2), 0, 0, 0};
    else w.s = FastmaxStrides{x.stride(1), x.stride(2), x.stride(0), static_cast<int32_t>(x.size(1)), 0};
    w.bh = x.size(0) * x.size(1); w.n = x.size(2); w.d = x.size(3);
  }
  return w;
}

// A new tensor shaped like `like` with n tokens; a 4-D view whose tokens lie outside its heads in
// memory (the projection layout (b, n, h, d)) gets its result in the same order, so the caller's
// transpose back to (b, n, h*d) is a view as well.
torch::Tensor empty_like_layout(const torch::Tensor& like, int64_t n, torch::ScalarType dtype) {
  if (like.dim() == 3) return torch::empty({like.size(0), n, like.size(2)}, like.options().dtype(dtype));
  const int64_t b = like.size(0), h = like.size(1), d = like.size(3);
  if (h > 1 && like.stride(2) > like.stride(1))
    return torch::empty({b, n, h, d}, like.options().dtype(dtype)).permute({0, 2, 1, 3});
  return torch::empty({b, h, n, d}, like.options().dtype(dtype));
}

FastmaxStrides gstrides_of(const torch::Tensor& g) {
  if (g.dim() == 3 && g.size(1) == 1) return FastmaxStrides{g.stride(0), g.stride(2), 0, 0, 0};
  if (g.dim() == 3) return FastmaxStrides{g.stride(1), g.stride(2), g.stride(0), static_cast<int32_t>(g.size(1)), 0};
  return FastmaxStrides{g.stride(0), g.stride(1), 0, 0, 0};
}

// Folded max-norm normalisation (FastmaxNormFold): the key tensors of maxnorm_stats, or undefined tensors for "off".
struct NormArgs {
  torch::Tensor q_keys, k_keys;
  double lim = 1.0;
  bool grad = false;
};

void apply_norm_args(FastmaxDesc& d, const NormArgs* na) {
  if (!na) return;
  auto check = [&](const torch::Tensor& t, int64_t n, const char* what) -> const void* {
    if (!t.defined()) return nullptr;
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kInt64 && t.is_contiguous() &&
                    t.numel() * 8 == int64_t(fastmax_maxnorm_stats_bytes(d.bh, static_cast<int32_t>(n))),
                what, " must be the int64 tensor maxnorm_stats returned for this tensor");
    return t.data_ptr();
  };
  d.norm.q_keys = check(na->q_keys, d.nq, "q_keys");
  d.norm.k_keys = check(na->k_keys, d.nk, "k_keys");
  d.norm.lim = float(na->lim);
  d.norm.grad = na->grad ? 1 : 0;
}

FastmaxDesc ex_desc(const View& q, const View& k, const View& v, bool mask, double inv_tau, double a0, double a1,
                    double a2, int64_t p, int64_t chunk, int64_t flags) {
  FM_CHECK_CUDA(q.t); FM_CHECK_CUDA(k.t); FM_CHECK_CUDA(v.t);
  TORCH_CHECK(k.bh == q.bh && v.bh == q.bh && k.d == q.d && v.d == q.d && v.n == k.n,
              "q, k, v must be (bh, nq, d), (bh, nk, d), (bh, nk, d)");
  TORCH_CHECK(k.t.scalar_type() == q.t.scalar_type() && v.t.scalar_type() == q.t.scalar_type(),
              "q, k, v must share one dtype");
  TORCH_CHECK(chunk >= 0 && chunk <= (int64_t(1) << 30), "chunk must be between 0 and 2^30, got ", chunk);
  TORCH_CHECK(flags >= 0 && flags <= 15, "unknown flags ", flags);
  TORCH_CHECK(q.bh <= 65535 && q.n <= (int64_t(1) << 30) && k.n <= (int64_t(1) << 30), "problem too large for 32-bit sizes");
  FastmaxDesc d{};
  d.bh = static_cast<int32_t>(q.bh); d.nq = static_cast<int32_t>(q.n); d.nk = static_cast<int32_t>(k.n);
  d.d = static_cast<int32_t>(q.d); d.dtype = dtype_code(q.t);
  d.mask = mask ? 1 : 0; d.p = static_cast<int32_t>(p);
  d.a0 = float(a0); d.a1 = float(a1); d.a2 = float(a2); d.inv_tau = float(inv_tau);
  d.chunk = static_cast<int32_t>(chunk); d.flags = static_cast<int32_t>(flags);
  d.sq = q.s; d.sk = k.s; d.sv = v.s;
  return d;
}

std::vector<torch::Tensor> forward_any(torch::Tensor q_, torch::Tensor k_, torch::Tensor v_, bool mask, double inv_tau,
                                       double a0, double a1, double a2, int64_t p, int64_t chunk, int64_t flags,
                                       const NormArgs* na = nullptr) {
  const View q = view_of(q_, "q"), k = view_of(k_, "k"), v = view_of(v_, "v");
  FastmaxDesc d = ex_desc(q, k, v, mask, inv_tau, a0, a1, a2, p, chunk, flags);
  apply_norm_args(d, na);
  torch::Tensor o = empty_like_layout(q.t, q.n, q.t.scalar_type());
  torch::Tensor g = q.t.dim() == 4 ? torch::empty({q.t.size(0), q.t.size(1), q.n}, q.t.options().dtype(torch::kFloat32))
                                   : torch::empty({q.bh, q.n}, q.t.options().dtype(torch::kFloat32));
  d.so = view_of(o, "o").s;
  d.sg = gstrides_of(g);
  size_t fwd = 0, bwd = 0;
  check_status(fastmax_workspace_bytes(&d, &fwd, &bwd), "fastmax_workspace_bytes");
  torch::Tensor ws = workspace(fwd, q.t);
  check_status(fastmax_forward(&d, q.t.data_ptr(), k.t.data_ptr(), v.t.data_ptr(), o.data_ptr(), g.data_ptr<float>(),
                               ws.data_ptr(), fwd, stream_of(q.t)), "fastmax_forward");
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
                                        int64_t flags, const NormArgs* na = nullptr) {
  const View q = view_of(q_, "q"), k = view_of(k_, "k"), v = view_of(v_, "v");
  const View o = view_of(o_, "o"), go = view_of(go_, "grad_output");
  FastmaxDesc d = ex_desc(q, k, v, mask, inv_tau, a0, a1, a2, p, chunk, flags);
  apply_norm_args(d, na);
  TORCH_CHECK(o.t.scalar_type() == q.t.scalar_type() && go.t.scalar_type() == q.t.scalar_type(),
              "o and grad_output must match q");
  TORCH_CHECK(o.bh == q.bh && o.n == q.n && o.d == q.d && go.bh == q.bh && go.n == q.n && go.d == q.d,
              "o and grad_output must be shaped like q");
  TORCH_CHECK(g_.scalar_type() == torch::kFloat32 && g_.numel() == int64_t(d.bh) * d.nq, "g must be float32 (bh, nq)");
  torch::Tensor g = g_.dim() == 3 ? g_ : g_.contiguous().view({d.bh, d.nq});
  torch::Tensor dq = empty_like_layout(q.t, q.n, q.t.scalar_type());
  torch::Tensor dk = empty_like_layout(k.t, k.n, q.t.scalar_type());
  torch::Tensor dv = empty_like_layout(v.t, v.n, q.t.scalar_type());
  d.so = o.s; d.sdo = go.s;
  d.sg = gstrides_of(g);
  d.sdq = view_of(dq, "dq").s; d.sdk = view_of(dk, "dk").s; d.sdv = view_of(dv, "dv").s;
  size_t fwd = 0, bwd = 0;
  check_status(fastmax_workspace_bytes(&d, &fwd, &bwd), "fastmax_workspace_bytes");
  torch::Tensor ws = workspace(bwd, q.t);
  // causal with more keys than queries keeps nothing from its forward: the plain backward runs
  if (saved && !(mask && k.n > q.n)) {
    TORCH_CHECK(saved->is_cuda() && saved->scalar_type() == torch::kUInt8 && saved->is_contiguous(),
                "saved workspace must be the uint8 tensor returned by forward_save");
    check_status(fastmax_backward_saved(&d, q.t.data_ptr(), k.t.data_ptr(), v.t.data_ptr(), o.t.data_ptr(),
                                        g.data_ptr<float>(), go.t.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                        dv.data_ptr(), saved->data_ptr(), size_t(saved->numel()), ws.data_ptr(), bwd,
                                        stream_of(q.t)),
                 "fastmax_backward_saved");
  } else {
    check_status(fastmax_backward(&d, q.t.data_ptr(), k.t.data_ptr(), v.t.data_ptr(), o.t.data_ptr(),
                                  g.data_ptr<float>(), go.t.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                  ws.data_ptr(), bwd, stream_of(q.t)), "fastmax_backward");
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

// Statistics of the folded max-norm normalisation for q and k in one launch (fastmax_maxnorm_stats): two int64
// tensors (bh, blocks of 256 tokens).
std::tuple<torch::Tensor, torch::Tensor> maxnorm_stats(torch::Tensor q_, torch::Tensor k_) {
  const View q = view_of(q_, "q"), k = view_of(k_, "k");
  FM_CHECK_CUDA(q.t); FM_CHECK_CUDA(k.t);
  TORCH_CHECK(k.bh == q.bh && k.d == q.d && k.t.scalar_type() == q.t.scalar_type(), "q and k must agree in batch*heads, head size and dtype");
  FastmaxNormDesc dq{}, dk{};
  dq.bh = static_cast<int32_t>(q.bh); dq.n = static_cast<int32_t>(q.n); dq.d = static_cast<int32_t>(q.d);
  dq.dtype = dtype_code(q.t); dq.sx = q.s;
  dk = dq; dk.n = static_cast<int32_t>(k.n); dk.sx = k.s;
  auto keys = [&](int32_t n) {
    return torch::empty({q.bh, int64_t(fastmax_maxnorm_stats_bytes(dq.bh, n) / 8 / q.bh)}, q.t.options().dtype(torch::kInt64));
  };
  torch::Tensor kq = keys(dq.n), kk = keys(dk.n);
  check_status(fastmax_maxnorm_stats(&dq, q.t.data_ptr(), kq.data_ptr(), &dk, k.t.data_ptr(), kk.data_ptr(), stream_of(q.t)),
               "fastmax_maxnorm_stats");
  return {kq, kk};
}

// Forward with q and k normalised on load (x_hat = lim * x / max-norm); keeps its workspace for backward_norm.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> forward_norm(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                                                                   torch::Tensor q_keys, torch::Tensor k_keys, double lim,
                                                                   bool mask, double inv_tau, double a0, double a1,
                                                                   double a2, int64_t p, int64_t chunk, int64_t flags) {
  NormArgs na{q_keys, k_keys, lim, false};
  std::vector<torch::Tensor> r = forward_any(q, k, v, mask, inv_tau, a0, a1, a2, p, chunk,
                                             flags | FASTMAX_FLAG_SAVE_FOR_BACKWARD, &na);
  return {r[0], r[1], r[2]};
}

// Its backward.  grad: true -> gradients with respect to the raw q and k (through the normalisation);
// false -> with respect to the normalised tensors (what the reference's extension returns).
std::vector<torch::Tensor> backward_norm(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor o, torch::Tensor g,
                                         torch::Tensor go, torch::Tensor saved, torch::Tensor q_keys, torch::Tensor k_keys,
                                         double lim, bool grad, bool mask, double inv_tau, double a0, double a1, double a2,
                                         int64_t p, int64_t chunk, int64_t flags) {
  NormArgs na{q_keys, k_keys, lim, grad};
  return backward_any(q, k, v, o, g, go, &saved, mask, inv_tau, a0, a1, a2, p, chunk,
                      flags | FASTMAX_FLAG_SAVE_FOR_BACKWARD, &na);
}

// Incremental decoding on a persistent moment state (fastmax_decode_* in the C header).
FastmaxDesc decode_desc(const View& q, const View& k, const View& v, double inv_tau, double a0, double a1, double a2,
                        int64_t p) {
  return ex_desc(q, k, v, true, inv_tau, a0, a1, a2, p, 0, 0);
}

// an empty state for keys shaped like k: zero-filled float32
torch::Tensor decode_state(torch::Tensor k_, double inv_tau, double a0, double a1, double a2, int64_t p) {
  const View k = view_of(k_, "k");
  FastmaxDesc d = decode_desc(k, k, k, inv_tau, a0, a1, a2, p);
  return torch::zeros({int64_t(fastmax_decode_state_bytes(&d) / 4)}, k.t.options().dtype(torch::kFloat32));
}

void decode_absorb(torch::Tensor k_, torch::Tensor v_, torch::Tensor state, double inv_tau, double a0, double a1, double a2,
                   int64_t p) {
  const View k = view_of(k_, "k"), v = view_of(v_, "v");
  FastmaxDesc d = decode_desc(k, k, v, inv_tau, a0, a1, a2, p);
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == torch::kFloat32 && state.is_contiguous() &&
                  size_t(state.numel()) * 4 == fastmax_decode_state_bytes(&d), "state must come from decode_state for this shape");
  check_status(fastmax_decode_absorb(&d, k.t.data_ptr(), v.t.data_ptr(), state.data_ptr<float>(), stream_of(k.t)),
               "fastmax_decode_absorb");
}

std::tuple<torch::Tensor, torch::Tensor> decode_step(torch::Tensor q_, torch::Tensor k_, torch::Tensor v_, torch::Tensor state,
                                                    double inv_tau, double a0, double a1, double a2, int64_t p) {
  const View q = view_of(q_, "q"), k = view_of(k_, "k"), v = view_of(v_, "v");
  TORCH_CHECK(q.n == 1 && k.n == 1, "decode_step takes one token");
  FastmaxDesc d = decode_desc(q, k, v, inv_tau, a0, a1, a2, p);
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == torch::kFloat32 && state.is_contiguous() &&
                  size_t(state.numel()) * 4 == fastmax_decode_state_bytes(&d), "state must come from decode_state for this shape");
  torch::Tensor o = empty_like_layout(q.t, 1, q.t.scalar_type());
  torch::Tensor g = q.t.dim() == 4 ? torch::empty({q.t.size(0), q.t.size(1), 1}, q.t.options().dtype(torch::kFloat32))
                                   : torch::empty({q.bh, 1}, q.t.options().dtype(torch::kFloat32));
  d.so = view_of(o, "o").s;
  d.sg = gstrides_of(g);
  torch::Tensor scratch = torch::empty({int64_t(fastmax_decode_scratch_bytes(&d) / 4)}, q.t.options().dtype(torch::kFloat32));
  check_status(fastmax_decode_step(&d, q.t.data_ptr(), k.t.data_ptr(), v.t.data_ptr(), state.data_ptr<float>(), o.data_ptr(),
                                   g.data_ptr<float>(), scratch.data_ptr<float>(), stream_of(q.t)), "fastmax_decode_step");
  return {o, g};
}

// y = scale * (x - centre) / max_n ||x_n - centre||  (see fastmax_normalize in the C header)
torch::Tensor normalize(torch::Tensor x_, int64_t centre, bool max_norm, double scale) {
  const View x = view_of(x_, "x");
  FM_CHECK_CUDA(x.t);
  FastmaxNormDesc nd{};
  nd.bh = static_cast<int32_t>(x.bh); nd.n = static_cast<int32_t>(x.n); nd.d = static_cast<int32_t>(x.d);
  nd.dtype = dtype_code(x.t); nd.centre = static_cast<int32_t>(centre); nd.max_norm = max_norm ? 1 : 0;
  nd.scale = float(scale);
  torch::Tensor y = empty_like_layout(x.t, x.n, x.t.scalar_type());
  nd.sx = x.s; nd.sy = view_of(y, "y").s;
  torch::Tensor stats = torch::empty({int64_t(fastmax_normalize_stats_bytes(&nd) / sizeof(float))},
                                     x.t.options().dtype(torch::kFloat32));
  check_status(fastmax_normalize(&nd, x.t.data_ptr(), y.data_ptr(), stats.data_ptr<float>(), stream_of(x.t)),
               "fastmax_normalize");
  return y;
}

// gradient of normalize() with respect to x (see fastmax_normalize_backward in the C header)
torch::Tensor normalize_backward(torch::Tensor x_, torch::Tensor dy_, int64_t centre, bool max_norm, double scale) {
  const View x = view_of(x_, "x");
  const View dy = view_of(dy_, "dy");
  FM_CHECK_CUDA(x.t);
  FM_CHECK_CUDA(dy.t);
  TORCH_CHECK(dy.bh == x.bh && dy.n == x.n && dy.d == x.d && dy.t.scalar_type() == x.t.scalar_type(),
              "dy must have x's shape and dtype");
  FastmaxNormDesc nd{};
  nd.bh = static_cast<int32_t>(x.bh); nd.n = static_cast<int32_t>(x.n); nd.d = static_cast<int32_t>(x.d);
  nd.dtype = dtype_code(x.t); nd.centre = static_cast<int32_t>(centre); nd.max_norm = max_norm ? 1 : 0;
  nd.scale = float(scale);
  // dx shares x's strides: lay it out like x, and if that is not possible take a packed copy of x
  torch::Tensor xs = x.t;
  torch::Tensor dx = empty_like_layout(xs, x.n, xs.scalar_type());
  View dxv = view_of(dx, "dx");
  View xv = x;
  if (dxv.s.bh != x.s.bh || dxv.s.n != x.s.n || dxv.s.b != x.s.b || dxv.s.heads != x.s.heads) {
    xs = x.t.contiguous();
    xv = view_of(xs, "x");
    dx = torch::empty_like(xs);
  }
  nd.sx = xv.s; nd.sy = dy.s;
  const size_t nbytes = fastmax_normalize_backward_stats_bytes(&nd);
  torch::Tensor stats = torch::empty({int64_t(nbytes / 4 + 1)}, x.t.options().dtype(torch::kFloat32));
  check_status(fastmax_normalize_backward(&nd, xs.data_ptr(), dy.t.data_ptr(), dx.data_ptr(), stats.data_ptr<float>(),
                                          stream_of(x.t)), "fastmax_normalize_backward");
  return dx;
}

// k + temperature * rpe[(l + n) % (2n - 1)]  (see fastmax_key_rpe in the C header)
torch::Tensor key_rpe(torch::Tensor k_, torch::Tensor rpe, double temperature) {
  const View k = view_of(k_, "k");
  FM_CHECK_CUDA(k.t);
  TORCH_CHECK(rpe.dim() == 2 && rpe.size(0) == 2 * k.n - 1 && rpe.size(1) == k.d, "rpe must be (2n-1, d) = (", 2 * k.n - 1,
              ", ", k.d, ")");
  torch::Tensor table = rpe.to(k.t.device(), torch::kFloat32).contiguous();
  FastmaxNormDesc nd{};
  nd.bh = static_cast<int32_t>(k.bh); nd.n = static_cast<int32_t>(k.n); nd.d = static_cast<int32_t>(k.d);
  nd.dtype = dtype_code(k.t);
  torch::Tensor y = empty_like_layout(k.t, k.n, k.t.scalar_type());
  nd.sx = k.s; nd.sy = view_of(y, "y").s;
  check_status(fastmax_key_rpe(&nd, k.t.data_ptr(), table.data_ptr<float>(), y.data_ptr(), float(temperature), stream_of(k.t)),
               "fastmax_key_rpe");
  return y;
}

// o * (1 + scale * noise)  (see fastmax_output_noise in the C header)
torch::Tensor output_noise(torch::Tensor o_, torch::Tensor noise_, double scale) {
  const View o = view_of(o_, "o");
  FM_CHECK_CUDA(o.t);
  TORCH_CHECK(noise_.sizes() == o_.sizes() && noise_.scalar_type() == o_.scalar_type() && noise_.device() == o_.device(),
              "noise must have o's shape, dtype and device");
  torch::Tensor noise = noise_.strides() == o.t.strides() ? noise_ : torch::empty_strided(o.t.sizes(), o.t.strides(), o.t.options()).copy_(noise_);
  FastmaxNormDesc nd{};
  nd.bh = static_cast<int32_t>(o.bh); nd.n = static_cast<int32_t>(o.n); nd.d = static_cast<int32_t>(o.d);
  nd.dtype = dtype_code(o.t);
  torch::Tensor y = empty_like_layout(o.t, o.n, o.t.scalar_type());
  nd.sx = o.s; nd.sy = view_of(y, "y").s;
  check_status(fastmax_output_noise(&nd, o.t.data_ptr(), noise.data_ptr(), y.data_ptr(), float(scale), stream_of(o.t)),
               "fastmax_output_noise");
  return y;
}

}  // namespace

PYBIND11_MODULE(fastmax_cuda, m) {
  m.def("forwardpass", &forwardpass, "forwardpass");
  m.def("backwardpass", &backwardpass, "backwardpass");
  m.def("forward_ex", &forward_ex, "strided forward: returns (o, g)");
  m.def("backward_ex", &backward_ex, "strided backward: returns [dq, dk, dv]");
  m.def("forward_save", &forward_save, "strided forward keeping its workspace: returns (o, g, saved)");
  m.def("backward_saved", &backward_saved, "strided backward on a saved forward workspace: returns [dq, dk, dv]");
  m.def("maxnorm_stats", &maxnorm_stats, "statistics of the folded max-norm normalisation of q and k: (q_keys, k_keys)");
  m.def("forward_norm", &forward_norm, "strided forward with q, k normalised on load: returns (o, g, saved)");
  m.def("backward_norm", &backward_norm, "backward of forward_norm: returns [dq, dk, dv]");
  m.def("decode_state", &decode_state, "empty decoding state (zeros) for keys shaped like k");
  m.def("decode_absorb", &decode_absorb, "add all tokens of k, v to a decoding state");
  m.def("decode_step", &decode_step, "one decoding step on the state: returns (o, g) of the new token");
  m.def("normalize", &normalize, "fused normalisation pass");
  m.def("normalize_backward", &normalize_backward, "gradient of the normalisation pass with respect to its input");
  m.def("key_rpe", &key_rpe, "keys with the relative-position rows added (the reference's commented-out step)");
  m.def("output_noise", &output_noise, "output times (1 + scale * noise) (the reference's apply_dropout)");
  m.def("version", []() { return fastmax_version(); });
}
