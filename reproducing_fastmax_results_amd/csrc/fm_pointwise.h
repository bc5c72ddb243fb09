// The two element-wise steps of the reference's forward_cuda that it ships switched off, as passes a caller
// can switch on:
//   * relative-position rows added to the keys after the temperature division
//     (apply_rpe_and_temp, fastmax_cuda_forward.cu:282-292; the addition at :289 is commented out there):
//       k[l][i][m] = k[l][i][m] / tau + rpe[(l + nk) % (2 nk - 1)][m]
//     Here the operator divides by tau inside its loads, so the pass writes k + tau * rpe.
//   * multiplicative noise on the output (apply_dropout, fastmax_cuda_forward.cu:340-349; called with
//     scale 0 at :443):  o[l][i][m] *= 1 + scale * noise[l][i][m].  The same pass applied to dO is its
//     backward.
// Both read one tensor (plus the table / the noise) and write one: HBM-bound, 16-byte accesses where the
// strides allow, 64 * FM_NORM_NP tokens of one batch*head per workgroup.
#pragma once
#include "fm_norm.h"

struct PointwiseArgs {
  int n;               // tokens
  int mode;            // 0: key RPE, 1: output noise
  float factor;        // tau (mode 0) or the noise scale (mode 1)
  const float* table;  // mode 0: (2 n - 1, d) contiguous fp32 rows
};

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_pointwise(TRef<const TIO> x, TRef<const TIO> noise, TRef<TIO> y, PointwiseArgs a) {
  constexpr int EPT = DH / 4, NP = FM_NORM_NP;
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok0 = FM_BID_X * 64 * NP + (tid >> 2), d0 = (tid & 3) * EPT;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p;
    if (tok >= a.n) continue;
    float v[EPT], w[EPT];
    fm_norm_load<TIO, DH>(x.base(bh) + int64_t(tok) * x.s_n, x.vec != 0, d0, v);
    if (a.mode == 0) {
      const float* row = a.table + int64_t((tok + a.n) % (2 * a.n - 1)) * DH + d0;
#pragma unroll
      for (int j = 0; j < EPT; ++j) v[j] += a.factor * row[j];
    } else {
      fm_norm_load<TIO, DH>(noise.base(bh) + int64_t(tok) * noise.s_n, noise.vec != 0, d0, w);
#pragma unroll
      for (int j = 0; j < EPT; ++j) v[j] *= 1.0f + a.factor * w[j];
    }
#pragma unroll
    for (int j = 0; j < EPT; j += 8) IO<TIO>::st8(y.base(bh) + int64_t(tok) * y.s_n + d0 + j, y.vec != 0, &v[j]);
  }
}

template <typename TIO, int DH>
int fm_pointwise_run(const FastmaxNormDesc* d, const void* x, const void* noise, void* y, const PointwiseArgs& a,
                     fm_stream_t stream) {
  const TRef<const TIO> xr = fm_ref<const TIO>(static_cast<const TIO*>(x), d->sx);
  const TRef<const TIO> nr = fm_ref<const TIO>(static_cast<const TIO*>(noise ? noise : x), d->sx);
  const TRef<TIO> yr = fm_ref<TIO>(static_cast<TIO*>(y), d->sy);
  const fm_dim3 grid(fm_norm_blocks(d->n), d->bh);
  FM_KERNEL_LAUNCH((k_pointwise<TIO, DH>), grid, fm_dim3(256), 0, stream, xr, nr, yr, a);
  return fm_after_launch() ? FASTMAX_ERR_LAUNCH : FASTMAX_OK;
}

inline int fm_pointwise_dispatch(const FastmaxNormDesc* d, const void* x, const void* noise, void* y, const PointwiseArgs& a,
                                 fm_stream_t stream) {
  if (!d || !x || !y) return FASTMAX_ERR_NULL;
  if (a.mode == 0 ? !a.table : !noise) return FASTMAX_ERR_NULL;
  if (d->dtype != FASTMAX_F32 && d->dtype != FASTMAX_BF16) return FASTMAX_ERR_DTYPE;
  if (d->bh <= 0 || d->n <= 0 || d->bh > 65535 || d->n > (1 << 30)) return FASTMAX_ERR_SHAPE;
  if (d->d != 32 && d->d != 64) return FASTMAX_ERR_UNSUPPORTED;
  if (d->sx.n < d->d || d->sy.n < d->d) return FASTMAX_ERR_SHAPE;
  if (d->dtype == FASTMAX_F32)
    return d->d == 64 ? fm_pointwise_run<float, 64>(d, x, noise, y, a, stream) : fm_pointwise_run<float, 32>(d, x, noise, y, a, stream);
  return d->d == 64 ? fm_pointwise_run<fm_bf16, 64>(d, x, noise, y, a, stream) : fm_pointwise_run<fm_bf16, 32>(d, x, noise, y, a, stream);
}
