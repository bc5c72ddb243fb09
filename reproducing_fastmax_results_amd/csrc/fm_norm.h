// Fused q/k normalisation pass (bandwidth bound).
//   y = scale * (x - centre) / max_n ||x_n - centre||_2      (max_norm)
//   y = scale * (x - centre)                                  (otherwise)
// centre: 0 none (transformer/model.py:97-102), 1 feature mean
// (fastattention_einops.py:327-334), 2 token mean (score_function.py:42-47).
// Replaces apply_rpe_and_temp / calc_norms / find_max / apply_norm
// (fastmax_cuda_forward.cu:282-338).  Reductions use no floating-point atomics:
// the maximum is taken with an integer atomicMax on the bit pattern of a
// non-negative float, which is order independent.
#pragma once
#include "fastmax_hip.h"
#include "fm_kernels.h"

// stats layout per batch*head: [0] max squared norm (as float bits), [1] unused, [2..2+d) token mean
template <int DH> struct NormStats { static constexpr int N = DH + 2; };

template <int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_clear(float* stats) {
  const int i = FM_BID_X * 256 + FM_TID_X;
  if (FM_TID_X < NormStats<DH>::N) stats[FM_BID_X * NormStats<DH>::N + FM_TID_X] = 0.f;
  (void)i;
}

// token mean per feature: one workgroup per (8 features, batch*head), 16-byte loads, a fixed
// reduction tree (the same sum order on every run).  grid (DH / 8, bh).
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_colmean(TRef<const TIO> x, int n, float* FM_RESTRICT out, int64_t out_stride) {
  FM_SHARED float part[8 * 256];
  const int tid = FM_TID_X, d0 = FM_BID_X * 8, bh = FM_BID_Y;
  float s[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) s[j] = 0.f;
  // eight rows in flight per thread (one row per trip left the kernel waiting on memory latency)
  for (int t = tid; t < n; t += 256 * 8) {
    float v[8][8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int tt = t + 256 * u;
      if (tt < n) {
        IO<TIO>::ld8(x.base(bh) + int64_t(tt) * x.s_n + d0, x.vec != 0, v[u]);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[u][j] = 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < 8; ++j) s[j] += v[u][j];
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) part[j * 256 + tid] = s[j];
  FM_SYNC();
  for (int stride = 128; stride > 0; stride >>= 1) {
    if (tid < stride) {
#pragma unroll
      for (int j = 0; j < 8; ++j) part[j * 256 + tid] += part[j * 256 + tid + stride];
    }
    FM_SYNC();
  }
  if (tid < 8) out[bh * out_stride + d0 + tid] = part[tid * 256] / float(n);   // out: DH means per batch*head
}

// A thread's quarter of one token row, and the centring of it (the feature mean needs the four
// threads of the token: every lane of the wavefront must call fm_norm_centre).
template <typename TIO, int DH>
FM_DEVICE void fm_norm_load(const TIO* row, bool vec, int d0, float v[DH / 4]) {
#pragma unroll
  for (int j = 0; j < DH / 4; j += 8) IO<TIO>::ld8(row + d0 + j, vec, &v[j]);
}
template <int DH>
FM_DEVICE void fm_norm_centre(float v[DH / 4], int d0, int centre, const float* mean) {
  constexpr int EPT = DH / 4;
  if (centre == 1) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < EPT; ++j) s += v[j];
    s += fm_shfl_xor(s, 1);
    s += fm_shfl_xor(s, 2);
    s *= 1.0f / float(DH);
#pragma unroll
    for (int j = 0; j < EPT; ++j) v[j] -= s;
  } else if (centre == 2) {
#pragma unroll
    for (int j = 0; j < EPT; ++j) v[j] -= mean[d0 + j];
  }
}
template <typename TIO, int DH>
FM_DEVICE void fm_norm_load_centred(const TIO* row, bool vec, int d0, int centre, const float* mean, float v[DH / 4]) {
  fm_norm_load<TIO, DH>(row, vec, d0, v);
  fm_norm_centre<DH>(v, d0, centre, mean);
}

// Token blocks of 64 (four threads per token) per workgroup in the kernels below: the loads of all
// its blocks are issued before the first is used, so a thread has NP * DH / 32 16-byte loads in flight.
static constexpr int FM_NORM_NP = 4;     // forward kernels and the backward's second pass
static constexpr int FM_NORMB_NP = 2;    // backward statistics (two tensors per token)

// grid (ceil(n / (64 * FM_NORM_NP)), bh); four threads per token
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_maxnorm(TRef<const TIO> x, int n, int centre, float* FM_RESTRICT stats) {
  constexpr int EPT = DH / 4, NP = FM_NORM_NP;
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok0 = FM_BID_X * 64 * NP + (tid >> 2), d0 = (tid & 3) * EPT;
  float* st = stats + bh * NormStats<DH>::N;
  float v[NP][EPT];
  // every lane takes part in the shuffles; rows past the end re-read the last row and count as zero
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p, tk = tok < n ? tok : n - 1;
    fm_norm_load<TIO, DH>(x.base(bh) + int64_t(tk) * x.s_n, x.vec != 0, d0, v[p]);
  }
  float mx = 0.f;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    fm_norm_centre<DH>(v[p], d0, centre, st + 2);
    float nrm = 0.f;
#pragma unroll
    for (int j = 0; j < EPT; ++j) nrm += v[p][j] * v[p][j];
    nrm += fm_shfl_xor(nrm, 1);
    nrm += fm_shfl_xor(nrm, 2);
    if (tok0 + 64 * p < n) mx = fm_fmaxf(mx, nrm);
  }
#pragma unroll
  for (int m = 4; m < 64; m <<= 1) mx = fm_fmaxf(mx, fm_shfl_xor(mx, m));
  if ((tid & 63) == 0) {
    uint32_t bits;
    __builtin_memcpy(&bits, &mx, 4);
#if defined(FM_HOSTSIM)
    uint32_t* p = reinterpret_cast<uint32_t*>(st);
    if (bits > *p) *p = bits;            // workgroups run one after another in the simulator
#else
    atomicMax(reinterpret_cast<unsigned int*>(st), bits);
#endif
  }
}

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_apply(TRef<const TIO> x, TRef<TIO> y, int n, int centre, int max_norm, float scale,
                                                  const float* FM_RESTRICT stats) {
  constexpr int EPT = DH / 4, NP = FM_NORM_NP;
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok0 = FM_BID_X * 64 * NP + (tid >> 2), d0 = (tid & 3) * EPT;
  const float* st = stats ? stats + bh * NormStats<DH>::N : nullptr;
  float v[NP][EPT];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p, tk = tok < n ? tok : n - 1;
    fm_norm_load<TIO, DH>(x.base(bh) + int64_t(tk) * x.s_n, x.vec != 0, d0, v[p]);
  }
  float f = scale;
  if (max_norm) f = scale / fm_sqrtf(st[0]);
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p;
    fm_norm_centre<DH>(v[p], d0, centre, st ? st + 2 : nullptr);
    if (tok < n) {
#pragma unroll
      for (int j = 0; j < EPT; ++j) v[p][j] *= f;
#pragma unroll
      for (int j = 0; j < EPT; j += 8) IO<TIO>::st8(y.base(bh) + int64_t(tok) * y.s_n + d0 + j, y.vec != 0, &v[p][j]);
    }
  }
}

template <typename TIO, int DH>
int fm_normalize_run(const FastmaxNormDesc* d, const void* x, void* y, float* stats, fm_stream_t stream) {
  const TRef<const TIO> xr = fm_ref<const TIO>(static_cast<const TIO*>(x), d->sx);
  const TRef<TIO> yr = fm_ref<TIO>(static_cast<TIO*>(y), d->sy);
  const fm_dim3 grid((d->n + 64 * FM_NORM_NP - 1) / (64 * FM_NORM_NP), d->bh);
  if (d->max_norm || d->centre == 2) {
    FM_KERNEL_LAUNCH((k_norm_clear<DH>), fm_dim3(d->bh), fm_dim3(256), 0, stream, stats);
    if (d->centre == 2)
      FM_KERNEL_LAUNCH((k_norm_colmean<TIO, DH>), fm_dim3(DH / 8, d->bh), fm_dim3(256), 0, stream, xr, d->n, stats + 2,
                       int64_t(NormStats<DH>::N));
    if (d->max_norm)
      FM_KERNEL_LAUNCH((k_norm_maxnorm<TIO, DH>), grid, fm_dim3(256), 0, stream, xr, d->n, d->centre, stats);
  }
  FM_KERNEL_LAUNCH((k_norm_apply<TIO, DH>), grid, fm_dim3(256), 0, stream, xr, yr, d->n, d->centre, d->max_norm,
                   d->scale, stats);
#if defined(FM_HOSTSIM)
  return FASTMAX_OK;
#else
  return hipGetLastError() == hipSuccess ? FASTMAX_OK : FASTMAX_ERR_LAUNCH;
#endif
}

inline int fm_normalize_dispatch(const FastmaxNormDesc* d, const void* x, void* y, float* stats, fm_stream_t stream) {
  if (!d || !x || !y) return FASTMAX_ERR_NULL;
  if (d->dtype != FASTMAX_F32 && d->dtype != FASTMAX_BF16) return FASTMAX_ERR_DTYPE;
  if (d->bh <= 0 || d->n <= 0 || d->bh > 65535) return FASTMAX_ERR_SHAPE;
  if (d->d != 32 && d->d != 64) return FASTMAX_ERR_UNSUPPORTED;
  if (d->centre < 0 || d->centre > 2) return FASTMAX_ERR_UNSUPPORTED;
  if ((d->max_norm || d->centre == 2) && !stats) return FASTMAX_ERR_WORKSPACE;
  if (d->sx.n < d->d || d->sy.n < d->d) return FASTMAX_ERR_SHAPE;
  if (d->dtype == FASTMAX_BF16) {
    return d->d == 64 ? fm_normalize_run<fm_bf16, 64>(d, x, y, stats, stream) : fm_normalize_run<fm_bf16, 32>(d, x, y, stats, stream);
  }
  return d->d == 64 ? fm_normalize_run<float, 64>(d, x, y, stats, stream) : fm_normalize_run<float, 32>(d, x, y, stats, stream);
}

// ------------------------------------------------------------------------------
// Backward of the pass above.  With c = x - centre, m = max_n ||c_n|| reached at token n*
// (the first one among equal norms), B = sum_{n,d} dy * c and C(.) the same centring applied to dy:
//   dx_n = (scale / m) * ( C(dy)_n - ([n == n*] - [centre == 2] / N) * (B / m^2) * c_{n*} )
// and dx = scale * C(dy) without max_norm.  The reference's extension drops this gradient
// (fastmax_cuda_backward.cu returns the gradients with respect to the normalised tensors); its
// Python variants carry it through autograd (score_function.py:40-55, fastattention_einops.py:327-334).
//
// stats per batch*head, fm_normb_stride(d, n) floats: [0..1] one 64-bit word, the bit pattern of the
// largest squared norm in the high half and ~token in the low half (an integer atomicMax finds
// the largest norm and, among equal ones, the first token); [2], [3] unused; [4 .. 4+d) token mean
// of x; [4+d .. 4+2d) token mean of dy; then one partial sum of dy * c per 64-token block, added
// in a fixed order by every workgroup of the second kernel (no floating-point atomics).
// ------------------------------------------------------------------------------
inline int64_t fm_normb_stride(int dh, int n) { return 4 + 2 * int64_t(dh) + ((n + 63) / 64 + 1) / 2 * 2; }

FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_normb_clear(float* stats, int64_t stride) {
  if (FM_TID_X < 4) stats[FM_BID_X * stride + FM_TID_X] = 0.f;
}

// grid (ceil(n / (64 * FM_NORMB_NP)), bh); four threads per token
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_normb_stats(TRef<const TIO> x, TRef<const TIO> dy, int n, int centre, int max_norm,
                                                   float* FM_RESTRICT stats, int64_t stride) {
  constexpr int EPT = DH / 4, NP = FM_NORMB_NP;
  FM_SHARED float wsum[NP][4];
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok0 = FM_BID_X * 64 * NP + (tid >> 2), d0 = (tid & 3) * EPT;
  float* st = stats + bh * stride;
  float c[NP][EPT], g[NP][EPT];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p, tk = tok < n ? tok : n - 1;
    fm_norm_load<TIO, DH>(x.base(bh) + int64_t(tk) * x.s_n, x.vec != 0, d0, c[p]);
    fm_norm_load<TIO, DH>(dy.base(bh) + int64_t(tk) * dy.s_n, dy.vec != 0, d0, g[p]);
  }
  float mx = -1.0f;
  int cand = 0x7fffffff;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p;
    fm_norm_centre<DH>(c[p], d0, centre, st + 4);
    float nrm = 0.f, b = 0.f;
#pragma unroll
    for (int j = 0; j < EPT; ++j) { nrm += c[p][j] * c[p][j]; b += g[p][j] * c[p][j]; }
    nrm += fm_shfl_xor(nrm, 1);
    nrm += fm_shfl_xor(nrm, 2);
    if (tok >= n) { nrm = -1.0f; b = 0.f; }
    if (nrm > mx) { mx = nrm; cand = tok; }            // blocks in ascending token order: the first token wins ties
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) b += fm_shfl_xor(b, m);
    if ((tid & 63) == 0) wsum[p][tid >> 6] = b;
  }
  // largest norm of the wavefront and, among equal ones, the first token
  float wmx = mx;
#pragma unroll
  for (int m = 4; m < 64; m <<= 1) wmx = fm_fmaxf(wmx, fm_shfl_xor(wmx, m));
  int wc = (mx == wmx && mx >= 0.f) ? cand : 0x7fffffff;
#pragma unroll
  for (int m = 4; m < 64; m <<= 1) { const int o = fm_shfl_xor_i(wc, m); wc = o < wc ? o : wc; }
  if ((tid & 63) == 0 && max_norm && wc != 0x7fffffff) {
    uint32_t bits;
    __builtin_memcpy(&bits, &wmx, 4);
    const unsigned long long key = (static_cast<unsigned long long>(bits) << 32) | uint32_t(~uint32_t(wc));
    unsigned long long* p = reinterpret_cast<unsigned long long*>(st);
#if defined(FM_HOSTSIM)
    if (key > *p) *p = key;              // workgroups run one after another in the simulator
#else
    atomicMax(p, key);
#endif
  }
  FM_SYNC();
  if (tid < NP && (FM_BID_X * NP + tid) * 64 < n)
    st[4 + 2 * DH + FM_BID_X * NP + tid] = (wsum[tid][0] + wsum[tid][1]) + (wsum[tid][2] + wsum[tid][3]);
}

// grid (ceil(n / (64 * FM_NORM_NP)), bh); four threads per token
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_normb_apply(TRef<const TIO> x, TRef<const TIO> dy, TRef<TIO> dx, int n, int centre,
                                                   int max_norm, float scale, const float* FM_RESTRICT stats, int64_t stride) {
  constexpr int EPT = DH / 4, NP = FM_NORM_NP;
  FM_SHARED float red[256];
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok0 = FM_BID_X * 64 * NP + (tid >> 2), d0 = (tid & 3) * EPT;
  const float* st = stats ? stats + bh * stride : nullptr;
  float g[NP][EPT];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p, tk = tok < n ? tok : n - 1;
    fm_norm_load<TIO, DH>(dy.base(bh) + int64_t(tk) * dy.s_n, dy.vec != 0, d0, g[p]);
  }
  float f = scale, kf = 0.f;
  int nstar = -1;
  float cs[EPT];
  if (max_norm) {
    const int nblk = (n + 63) / 64;
    float s = 0.f;
    for (int i = tid; i < nblk; i += 256) s += st[4 + 2 * DH + i];
    red[tid] = s;
    FM_SYNC();
    for (int w = 128; w > 0; w >>= 1) {
      if (tid < w) red[tid] += red[tid + w];
      FM_SYNC();
    }
    const unsigned long long key = *reinterpret_cast<const unsigned long long*>(st);
    const uint32_t bits = uint32_t(key >> 32);
    float m2;
    __builtin_memcpy(&m2, &bits, 4);
    nstar = int(~uint32_t(key));
    if (nstar < 0 || nstar >= n) nstar = 0;            // no token won (every norm is a NaN)
    f = scale / fm_sqrtf(m2);
    kf = red[0] / m2;
    // every lane takes part in the shuffles of the centring
    fm_norm_load_centred<TIO, DH>(x.base(bh) + int64_t(nstar) * x.s_n, x.vec != 0, d0, centre, st + 4, cs);
  }
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p;
    fm_norm_centre<DH>(g[p], d0, centre, st ? st + 4 + DH : nullptr);
    if (max_norm) {
      const float w = kf * ((tok == nstar ? 1.0f : 0.0f) - (centre == 2 ? 1.0f / float(n) : 0.0f));
#pragma unroll
      for (int j = 0; j < EPT; ++j) g[p][j] -= w * cs[j];
    }
    if (tok < n) {
#pragma unroll
      for (int j = 0; j < EPT; ++j) g[p][j] *= f;
#pragma unroll
      for (int j = 0; j < EPT; j += 8) IO<TIO>::st8(dx.base(bh) + int64_t(tok) * dx.s_n + d0 + j, dx.vec != 0, &g[p][j]);
    }
  }
}

template <typename TIO, int DH>
int fm_normalize_bwd_run(const FastmaxNormDesc* d, const void* x, const void* dy, void* dx, float* stats, fm_stream_t stream) {
  const TRef<const TIO> xr = fm_ref<const TIO>(static_cast<const TIO*>(x), d->sx);
  const TRef<const TIO> gr = fm_ref<const TIO>(static_cast<const TIO*>(dy), d->sy);
  const TRef<TIO> dxr = fm_ref<TIO>(static_cast<TIO*>(dx), d->sx);
  const fm_dim3 grid_stats((d->n + 64 * FM_NORMB_NP - 1) / (64 * FM_NORMB_NP), d->bh);
  const fm_dim3 grid((d->n + 64 * FM_NORM_NP - 1) / (64 * FM_NORM_NP), d->bh);
  const int64_t stride = fm_normb_stride(DH, d->n);
  if (d->max_norm || d->centre == 2) {
    FM_KERNEL_LAUNCH(k_normb_clear, fm_dim3(d->bh), fm_dim3(64), 0, stream, stats, stride);
    if (d->centre == 2) {
      FM_KERNEL_LAUNCH((k_norm_colmean<TIO, DH>), fm_dim3(DH / 8, d->bh), fm_dim3(256), 0, stream, xr, d->n, stats + 4, stride);
      FM_KERNEL_LAUNCH((k_norm_colmean<TIO, DH>), fm_dim3(DH / 8, d->bh), fm_dim3(256), 0, stream, gr, d->n, stats + 4 + DH,
                       stride);
    }
    if (d->max_norm)
      FM_KERNEL_LAUNCH((k_normb_stats<TIO, DH>), grid_stats, fm_dim3(256), 0, stream, xr, gr, d->n, d->centre, d->max_norm, stats,
                       stride);
  }
  FM_KERNEL_LAUNCH((k_normb_apply<TIO, DH>), grid, fm_dim3(256), 0, stream, xr, gr, dxr, d->n, d->centre, d->max_norm,
                   d->scale, stats, stride);
#if defined(FM_HOSTSIM)
  return FASTMAX_OK;
#else
  return hipGetLastError() == hipSuccess ? FASTMAX_OK : FASTMAX_ERR_LAUNCH;
#endif
}

inline int fm_normalize_bwd_dispatch(const FastmaxNormDesc* d, const void* x, const void* dy, void* dx, float* stats,
                                     fm_stream_t stream) {
  if (!d || !x || !dy || !dx) return FASTMAX_ERR_NULL;
  if (d->dtype != FASTMAX_F32 && d->dtype != FASTMAX_BF16) return FASTMAX_ERR_DTYPE;
  if (d->bh <= 0 || d->n <= 0 || d->bh > 65535) return FASTMAX_ERR_SHAPE;
  if (d->d != 32 && d->d != 64) return FASTMAX_ERR_UNSUPPORTED;
  if (d->centre < 0 || d->centre > 2) return FASTMAX_ERR_UNSUPPORTED;
  if ((d->max_norm || d->centre == 2) && !stats) return FASTMAX_ERR_WORKSPACE;
  if (d->sx.n < d->d || d->sy.n < d->d) return FASTMAX_ERR_SHAPE;
  if (d->dtype == FASTMAX_BF16) {
    return d->d == 64 ? fm_normalize_bwd_run<fm_bf16, 64>(d, x, dy, dx, stats, stream)
                      : fm_normalize_bwd_run<fm_bf16, 32>(d, x, dy, dx, stats, stream);
  }
  return d->d == 64 ? fm_normalize_bwd_run<float, 64>(d, x, dy, dx, stats, stream)
                    : fm_normalize_bwd_run<float, 32>(d, x, dy, dx, stats, stream);
}
