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
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_colmean(TRef<const TIO> x, int n, float* FM_RESTRICT stats) {
  FM_SHARED float part[8 * 256];
  const int tid = FM_TID_X, d0 = FM_BID_X * 8, bh = FM_BID_Y;
  float s[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) s[j] = 0.f;
  for (int t = tid; t < n; t += 256) {
    float v[8];
    IO<TIO>::ld8(x.base(bh) + int64_t(t) * x.s_n + d0, x.vec != 0, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) s[j] += v[j];
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
  if (tid < 8) stats[bh * NormStats<DH>::N + 2 + d0 + tid] = part[tid * 256] / float(n);
}

template <typename TIO, int DH>
FM_DEVICE void fm_norm_load_centred(const TIO* row, bool vec, int d0, int centre, const float* mean, float v[DH / 4]) {
  constexpr int EPT = DH / 4;
#pragma unroll
  for (int j = 0; j < EPT; j += 8) IO<TIO>::ld8(row + d0 + j, vec, &v[j]);
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

// grid (ceil(n/64), bh); four threads per token
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_maxnorm(TRef<const TIO> x, int n, int centre, float* FM_RESTRICT stats) {
  constexpr int EPT = DH / 4;
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok = FM_BID_X * 64 + (tid >> 2), d0 = (tid & 3) * EPT;
  float* st = stats + bh * NormStats<DH>::N;
  float nrm = 0.f;
  // every lane takes part in the shuffles; rows past the end contribute zero
  const int tk = tok < n ? tok : n - 1;
  float v[EPT];
  fm_norm_load_centred<TIO, DH>(x.base(bh) + int64_t(tk) * x.s_n, x.vec != 0, d0, centre, st + 2, v);
#pragma unroll
  for (int j = 0; j < EPT; ++j) nrm += v[j] * v[j];
  nrm += fm_shfl_xor(nrm, 1);
  nrm += fm_shfl_xor(nrm, 2);
  if (tok >= n) nrm = 0.f;
#pragma unroll
  for (int m = 4; m < 64; m <<= 1) nrm = fm_fmaxf(nrm, fm_shfl_xor(nrm, m));
  if ((tid & 63) == 0) {
    uint32_t bits;
    __builtin_memcpy(&bits, &nrm, 4);
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
  constexpr int EPT = DH / 4;
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok = FM_BID_X * 64 + (tid >> 2), d0 = (tid & 3) * EPT;
  const float* st = stats ? stats + bh * NormStats<DH>::N : nullptr;
  const int tk = tok < n ? tok : n - 1;
  float v[EPT];
  fm_norm_load_centred<TIO, DH>(x.base(bh) + int64_t(tk) * x.s_n, x.vec != 0, d0, centre, st ? st + 2 : nullptr, v);
  float f = scale;
  if (max_norm) f = scale / fm_sqrtf(st[0]);
  if (tok < n) {
#pragma unroll
    for (int j = 0; j < EPT; ++j) v[j] *= f;
#pragma unroll
    for (int j = 0; j < EPT; j += 8) IO<TIO>::st8(y.base(bh) + int64_t(tok) * y.s_n + d0 + j, y.vec != 0, &v[j]);
  }
}

template <typename TIO, int DH>
int fm_normalize_run(const FastmaxNormDesc* d, const void* x, void* y, float* stats, fm_stream_t stream) {
  const TRef<const TIO> xr = fm_ref<const TIO>(static_cast<const TIO*>(x), d->sx);
  const TRef<TIO> yr = fm_ref<TIO>(static_cast<TIO*>(y), d->sy);
  const fm_dim3 grid((d->n + 63) / 64, d->bh);
  if (d->max_norm || d->centre == 2) {
    FM_KERNEL_LAUNCH((k_norm_clear<DH>), fm_dim3(d->bh), fm_dim3(256), 0, stream, stats);
    if (d->centre == 2)
      FM_KERNEL_LAUNCH((k_norm_colmean<TIO, DH>), fm_dim3(DH / 8, d->bh), fm_dim3(256), 0, stream, xr, d->n, stats);
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
