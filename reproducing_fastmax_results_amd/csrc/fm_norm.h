// Fused q/k normalisation pass (bandwidth bound).
//   y = scale * (x - centre) / max_n ||x_n - centre||_2      (max_norm)
//   y = scale * (x - centre)                                  (otherwise)
// centre: 0 none (transformer/model.py:97-102), 1 feature mean
// (fastattention_einops.py:327-334), 2 token mean (score_function.py:42-47).
// Replaces apply_rpe_and_temp / calc_norms / find_max / apply_norm
// (fastmax_cuda_forward.cu:282-338).  Reductions use no atomics at all: every workgroup leaves
// its partial result (largest squared norm, column sums) in the scratch buffer and the consumers add
// or compare the partials in a fixed order, so the result is the same bit pattern on every run.
#pragma once
#include "fastmax_hip.h"
#include "fm_kernels.h"

// Token blocks of 64 (four threads per token) per workgroup in the kernels below: the loads of all
// its blocks are issued before the first is used, so a thread has NP * DH / 32 16-byte loads in flight.
static constexpr int FM_NORM_NP = 4;     // forward kernels and the backward's second pass
static constexpr int FM_NORMB_NP = 2;    // backward statistics (two tensors per token)
// A slice whose largest squared norm is not above this value (all zeros: padding) comes out as zeros, with
// zero gradient, instead of 0 / 0.  (The reference's CUDA kernel floors at 0.1, fastmax_cuda_forward.cu:333;
// its Python variants do not floor at all; anything that is not an all-zero slice is far above this value.)
static constexpr float FM_NORM_FLOOR = 1e-30f;

// forward scratch per batch*head (floats): [0], [1] unused; [2 .. 2+d) token mean; then one largest
// squared norm per workgroup of k_norm_maxnorm; then, with the token-mean centring, d column sums per
// workgroup of k_norm_colsum
inline int fm_norm_blocks(int n) { return (n + 64 * FM_NORM_NP - 1) / (64 * FM_NORM_NP); }
inline int64_t fm_norm_stride(int dh, int n, int centre) {
  const int64_t nb = fm_norm_blocks(n);
  return (2 + int64_t(dh) + nb + (centre == 2 ? nb * dh : 0) + 1) / 2 * 2;
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

// Column sums over the workgroup's 64 * FM_NORM_NP tokens -> out[bh][block][DH]; k_norm_colfinal adds the
// blocks in a fixed order and divides.  grid (blocks, bh, tensors) and (bh, tensors).
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_colsum(TRef<const TIO> x0, TRef<const TIO> x1, int n, float* FM_RESTRICT out,
                                                   int64_t out_stride) {
  constexpr int EPT = DH / 4, NP = FM_NORM_NP;
  FM_SHARED float part[64 * (DH + 1)];
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const TRef<const TIO> x = FM_BID_Z ? x1 : x0;     // grid z: which tensor
  out += int64_t(FM_BID_Z) * FM_GDIM_X * DH;
  const int tok0 = FM_BID_X * 64 * NP + (tid >> 2), d0 = (tid & 3) * EPT;
  float v[NP][EPT];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p;
    if (tok < n) {
      fm_norm_load<TIO, DH>(x.base(bh) + int64_t(tok) * x.s_n, x.vec != 0, d0, v[p]);
    } else {
#pragma unroll
      for (int j = 0; j < EPT; ++j) v[p][j] = 0.f;
    }
  }
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    float a = 0.f;
#pragma unroll
    for (int p = 0; p < NP; ++p) a += v[p][j];
    part[(tid >> 2) * (DH + 1) + d0 + j] = a;
  }
  FM_SYNC();
  if (tid < DH) {
    float a = 0.f;
    for (int r = 0; r < 64; ++r) a += part[r * (DH + 1) + tid];
    out[bh * out_stride + int64_t(FM_BID_X) * DH + tid] = a;
  }
}
template <int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_colfinal(const float* FM_RESTRICT sums, int64_t sums_stride, int nblk, int n,
                                                     float* FM_RESTRICT mean, int64_t mean_stride) {
  constexpr int G = 256 / DH;                 // groups of DH threads, each takes every G-th block
  FM_SHARED float part[256];
  const int tid = FM_TID_X, bh = FM_BID_X, which = FM_BID_Y;     // which: tensor (sums and means of several lie side by side)
  const int g = tid / DH, f = tid % DH;
  sums += bh * sums_stride + int64_t(which) * nblk * DH;
  float a = 0.f;
  int b = g;
  for (; b + 3 * G < nblk; b += 4 * G) {      // four loads in flight
    const float v0 = sums[int64_t(b) * DH + f], v1 = sums[int64_t(b + G) * DH + f];
    const float v2 = sums[int64_t(b + 2 * G) * DH + f], v3 = sums[int64_t(b + 3 * G) * DH + f];
    a += v0; a += v1; a += v2; a += v3;
  }
  for (; b < nblk; b += G) a += sums[int64_t(b) * DH + f];
  part[tid] = a;
  FM_SYNC();
  if (tid < DH) {
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < G; ++i) t += part[i * DH + tid];
    mean[bh * mean_stride + which * DH + tid] = t / float(n);
  }
}

// grid (ceil(n / (64 * FM_NORM_NP)), bh); four threads per token
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_maxnorm(TRef<const TIO> x, int n, int centre, float* FM_RESTRICT stats, int64_t stride) {
  constexpr int EPT = DH / 4, NP = FM_NORM_NP;
  FM_SHARED float wmax[4];
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok0 = FM_BID_X * 64 * NP + (tid >> 2), d0 = (tid & 3) * EPT;
  float* st = stats + bh * stride;
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
  if ((tid & 63) == 0) wmax[tid >> 6] = mx;
  FM_SYNC();
  if (tid == 0) st[2 + DH + FM_BID_X] = fm_fmaxf(fm_fmaxf(wmax[0], wmax[1]), fm_fmaxf(wmax[2], wmax[3]));
}

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_norm_apply(TRef<const TIO> x, TRef<TIO> y, int n, int centre, int max_norm, float scale,
                                                  const float* FM_RESTRICT stats, int64_t stride) {
  constexpr int EPT = DH / 4, NP = FM_NORM_NP;
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok0 = FM_BID_X * 64 * NP + (tid >> 2), d0 = (tid & 3) * EPT;
  const float* st = stats ? stats + bh * stride : nullptr;
  float v[NP][EPT];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p, tk = tok < n ? tok : n - 1;
    fm_norm_load<TIO, DH>(x.base(bh) + int64_t(tk) * x.s_n, x.vec != 0, d0, v[p]);
  }
  float f = scale;
  if (max_norm) {
    // the largest of the workgroups' maxima: every lane takes a share, a butterfly joins them
    const int nblk = int(FM_GDIM_X);
    float m2 = 0.f;
    for (int b = tid & 63; b < nblk; b += 64) m2 = fm_fmaxf(m2, st[2 + DH + b]);
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) m2 = fm_fmaxf(m2, fm_shfl_xor(m2, m));
    f = m2 > FM_NORM_FLOOR ? scale / fm_sqrtf(m2) : 0.0f;
  }
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
  const int64_t stride = fm_norm_stride(DH, d->n, d->centre);
  if (d->centre == 2) {
    float* sums = stats + 2 + DH + grid.x;
    FM_KERNEL_LAUNCH((k_norm_colsum<TIO, DH>), grid, fm_dim3(256), 0, stream, xr, xr, d->n, sums, stride);
    FM_KERNEL_LAUNCH((k_norm_colfinal<DH>), fm_dim3(d->bh), fm_dim3(256), 0, stream, sums, stride, int(grid.x), d->n, stats + 2,
                     stride);
  }
  if (d->max_norm)
    FM_KERNEL_LAUNCH((k_norm_maxnorm<TIO, DH>), grid, fm_dim3(256), 0, stream, xr, d->n, d->centre, stats, stride);
  FM_KERNEL_LAUNCH((k_norm_apply<TIO, DH>), grid, fm_dim3(256), 0, stream, xr, yr, d->n, d->centre, d->max_norm,
                   d->scale, stats, stride);
  return fm_after_launch() ? FASTMAX_ERR_LAUNCH : FASTMAX_OK;
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
// stats per batch*head, fm_normb_stride(d, n, centre) floats: [0 .. 4) unused; [4 .. 4+d) token mean of x;
// [4+d .. 4+2d) token mean of dy; one partial sum of dy * c per 64-token block; one 64-bit key per
// workgroup of the statistics kernel (the bit pattern of its largest squared norm in the high half and
// ~token in the low half, so that an integer maximum finds the largest norm and, among equal ones, the
// first token); with the token-mean centring, the column sums of x and of dy per workgroup of
// k_norm_colsum.  Every workgroup of the second kernel joins the partials in the same fixed order:
// no atomics, nothing to clear, the same bits on every run.
// ------------------------------------------------------------------------------
FM_HOST_DEVICE inline int fm_normb_blocks(int n) { return (n + 64 * FM_NORMB_NP - 1) / (64 * FM_NORMB_NP); }
FM_HOST_DEVICE inline int64_t fm_normb_keys(int dh, int n) { return 4 + 2 * int64_t(dh) + ((n + 63) / 64 + 1) / 2 * 2; }
inline int64_t fm_normb_base(int dh, int n) { return fm_normb_keys(dh, n) + 2 * int64_t(fm_normb_blocks(n)); }
// with the token-mean centring the column sums of x and of dy per workgroup of k_norm_colsum follow
inline int64_t fm_normb_stride(int dh, int n, int centre) {
  return fm_normb_base(dh, n) + (centre == 2 ? 2 * int64_t(fm_norm_blocks(n)) * dh : 0);
}

// grid (ceil(n / (64 * FM_NORMB_NP)), bh); four threads per token
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_normb_stats(TRef<const TIO> x, TRef<const TIO> dy, int n, int centre, int max_norm,
                                                   float* FM_RESTRICT stats, int64_t stride) {
  constexpr int EPT = DH / 4, NP = FM_NORMB_NP;
  FM_SHARED float wsum[NP][4];
  FM_SHARED unsigned long long wkey[4];
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
  if ((tid & 63) == 0) {
    unsigned long long key = 0;          // no token of this wavefront has a norm that compares (all NaN)
    if (wc != 0x7fffffff) {
      uint32_t bits;
      __builtin_memcpy(&bits, &wmx, 4);
      key = (static_cast<unsigned long long>(bits) << 32) | uint32_t(~uint32_t(wc));
    }
    wkey[tid >> 6] = key;
  }
  FM_SYNC();
  if (tid < NP && (FM_BID_X * NP + tid) * 64 < n)
    st[4 + 2 * DH + FM_BID_X * NP + tid] = (wsum[tid][0] + wsum[tid][1]) + (wsum[tid][2] + wsum[tid][3]);
  if (tid == 64) {
    const unsigned long long a = wkey[0] > wkey[1] ? wkey[0] : wkey[1], b = wkey[2] > wkey[3] ? wkey[2] : wkey[3];
    reinterpret_cast<unsigned long long*>(st + fm_normb_keys(DH, n))[FM_BID_X] = a > b ? a : b;
  }
}

// grid (ceil(n / (64 * FM_NORM_NP)), bh); four threads per token
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_normb_apply(TRef<const TIO> x, TRef<const TIO> dy, TRef<TIO> dx, int n, int centre,
                                                   int max_norm, float scale, const float* FM_RESTRICT stats, int64_t stride) {
  constexpr int EPT = DH / 4, NP = FM_NORM_NP;
  FM_SHARED float red[256];
  FM_SHARED unsigned long long redk[256];
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
    // the largest key of the statistics kernel's workgroups: largest norm, first token among equal ones
    const unsigned long long* keys = reinterpret_cast<const unsigned long long*>(st + fm_normb_keys(DH, n));
    const int nkeys = fm_normb_blocks(n);
    unsigned long long kmax = 0;
    for (int i = tid; i < nkeys; i += 256) { const unsigned long long k = keys[i]; kmax = k > kmax ? k : kmax; }
    redk[tid] = kmax;
    FM_SYNC();
    for (int w = 128; w > 0; w >>= 1) {
      if (tid < w) {
        red[tid] += red[tid + w];
        redk[tid] = redk[tid + w] > redk[tid] ? redk[tid + w] : redk[tid];
      }
      FM_SYNC();
    }
    const unsigned long long key = redk[0];
    const uint32_t bits = uint32_t(key >> 32);
    float m2;
    __builtin_memcpy(&m2, &bits, 4);
    nstar = int(~uint32_t(key));
    if (nstar < 0 || nstar >= n) nstar = 0;            // no token won (every norm is a NaN)
    const bool some = m2 > FM_NORM_FLOOR;
    f = some ? scale / fm_sqrtf(m2) : 0.0f;
    kf = some ? red[0] / m2 : 0.0f;
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
  const int64_t stride = fm_normb_stride(DH, d->n, d->centre);
  if (d->max_norm || d->centre == 2) {
    if (d->centre == 2) {
      // the means of x and of dy lie side by side: one launch of the last step covers both
      float* sums = stats + fm_normb_base(DH, d->n);
      FM_KERNEL_LAUNCH((k_norm_colsum<TIO, DH>), fm_dim3(grid.x, grid.y, 2), fm_dim3(256), 0, stream, xr, gr, d->n, sums, stride);
      FM_KERNEL_LAUNCH((k_norm_colfinal<DH>), fm_dim3(d->bh, 2), fm_dim3(256), 0, stream, sums, stride, int(grid.x), d->n,
                       stats + 4, stride);
    }
    if (d->max_norm)
      FM_KERNEL_LAUNCH((k_normb_stats<TIO, DH>), grid_stats, fm_dim3(256), 0, stream, xr, gr, d->n, d->centre, d->max_norm, stats,
                       stride);
  }
  FM_KERNEL_LAUNCH((k_normb_apply<TIO, DH>), grid, fm_dim3(256), 0, stream, xr, gr, dxr, d->n, d->centre, d->max_norm,
                   d->scale, stats, stride);
  return fm_after_launch() ? FASTMAX_ERR_LAUNCH : FASTMAX_OK;
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

// ------------------------------------------------------------------------------
// The max-norm normalisation folded into the attention kernels (NormFold in fm_kernels.h): the one pass that
// is left reads the tensor once.  k_maxnorm_keys: grid (ceil(n / 256), bh, tensors); four threads per token;
// one 64-bit key per workgroup (bits of its largest squared token norm, ~token).  Two tensors (q and k) go
// in one launch.
// ------------------------------------------------------------------------------
template <typename TIO> struct MaxnormJob { TRef<const TIO> x; unsigned long long* keys; int n; int nblk; };

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_maxnorm_keys(MaxnormJob<TIO> j0, MaxnormJob<TIO> j1) {
  constexpr int EPT = DH / 4, NP = FM_MAXNORM_TOKENS / 64;
  FM_SHARED unsigned long long wkey[4];
  const MaxnormJob<TIO> J = FM_BID_Z ? j1 : j0;
  const int tid = FM_TID_X, bh = FM_BID_Y;
  if (int(FM_BID_X) >= J.nblk) return;                  // the shorter tensor of the two (workgroup-uniform)
  const int n = J.n;
  const int tok0 = FM_BID_X * FM_MAXNORM_TOKENS + (tid >> 2), d0 = (tid & 3) * EPT;
  float v[NP][EPT];
  // every lane takes part in the shuffles; rows past the end re-read the last row and do not count
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p, tk = tok < n ? tok : n - 1;
    fm_norm_load<TIO, DH>(J.x.base(bh) + int64_t(tk) * J.x.s_n, J.x.vec != 0, d0, v[p]);
  }
  float mx = -1.0f;
  int cand = 0x7fffffff;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    float nrm = 0.f;
#pragma unroll
    for (int j = 0; j < EPT; ++j) nrm += v[p][j] * v[p][j];
    nrm += fm_shfl_xor(nrm, 1);
    nrm += fm_shfl_xor(nrm, 2);
    const int tok = tok0 + 64 * p;
    if (tok >= n) nrm = -1.0f;
    if (nrm > mx) { mx = nrm; cand = tok; }             // ascending token order: the first token wins ties
  }
  float wmx = mx;
#pragma unroll
  for (int m = 4; m < 64; m <<= 1) wmx = fm_fmaxf(wmx, fm_shfl_xor(wmx, m));
  int wc = (mx == wmx && mx >= 0.f) ? cand : 0x7fffffff;
#pragma unroll
  for (int m = 4; m < 64; m <<= 1) { const int o = fm_shfl_xor_i(wc, m); wc = o < wc ? o : wc; }
  if ((tid & 63) == 0) {
    unsigned long long key = 0;                          // no norm of this wavefront compares (all NaN)
    if (wc != 0x7fffffff) {
      uint32_t bits;
      __builtin_memcpy(&bits, &wmx, 4);
      key = (static_cast<unsigned long long>(bits) << 32) | uint32_t(~uint32_t(wc));
    }
    wkey[tid >> 6] = key;
  }
  FM_SYNC();
  if (tid == 0) {
    const unsigned long long a = wkey[0] > wkey[1] ? wkey[0] : wkey[1], b = wkey[2] > wkey[3] ? wkey[2] : wkey[3];
    J.keys[int64_t(bh) * J.nblk + FM_BID_X] = a > b ? a : b;
  }
}

// The rank-one term of the normalisation's Jacobian.  With y = (lim / m) x, m = ||x_n*|| the largest token norm,
// dy the gradient with respect to y and B = sum_{n,d} dy * y over the whole slice:
//     dx_n = (lim / m) dy_n - [n == n*] * B * x_n* / m^2 .
// The attention kernels have stored (lim / m) dy and left B in parts (one per workgroup, added here in a fixed
// order); this kernel corrects the one row n*.  grid (bh, tensors), 64 threads.
template <typename TIO> struct NormFixJob {
  TRef<const TIO> x; TRef<TIO> dx; const unsigned long long* keys; int nblk; const float* bpart; int nb; int n;
};
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(64) k_norm_fix(NormFixJob<TIO> j0, NormFixJob<TIO> j1) {
  const NormFixJob<TIO> J = FM_BID_Y ? j1 : j0;
  const int lane = FM_TID_X, bh = FM_BID_X;
  if (!J.keys) return;
  float m2; int nstar;
  fm_maxnorm_join(J.keys + int64_t(bh) * J.nblk, J.nblk, lane, m2, nstar);
  if (!(m2 > FM_MAXNORM_FLOOR) || nstar < 0 || nstar >= J.n) return;
  // the parts in a fixed order: lane l adds parts l, l + 64, ...; then the lanes pairwise
  float b = 0.f;
  for (int i = lane; i < J.nb; i += 64) b += J.bpart[int64_t(bh) * J.nb + i];
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) b += fm_shfl_xor(b, m);
  if (lane < DH) {
    const float xv = IO<TIO>::ld(J.x.base(bh) + int64_t(nstar) * J.x.s_n + lane);
    TIO* p = J.dx.base(bh) + int64_t(nstar) * J.dx.s_n + lane;
    IO<TIO>::st(p, IO<TIO>::ld(p) - b * xv / m2);
  }
}

template <typename TIO, int DH>
int fm_maxnorm_run(const FastmaxNormDesc* d0, const void* x0, void* keys0, const FastmaxNormDesc* d1, const void* x1,
                   void* keys1, fm_stream_t stream) {
  MaxnormJob<TIO> j0{fm_ref<const TIO>(static_cast<const TIO*>(x0), d0->sx), static_cast<unsigned long long*>(keys0), d0->n,
                     fm_maxnorm_blocks(d0->n)};
  MaxnormJob<TIO> j1 = j0;
  if (d1) j1 = MaxnormJob<TIO>{fm_ref<const TIO>(static_cast<const TIO*>(x1), d1->sx), static_cast<unsigned long long*>(keys1),
                               d1->n, fm_maxnorm_blocks(d1->n)};
  const int nb = j0.nblk > j1.nblk ? j0.nblk : j1.nblk;
  FM_KERNEL_LAUNCH((k_maxnorm_keys<TIO, DH>), fm_dim3(nb, d0->bh, d1 ? 2 : 1), fm_dim3(256), 0, stream, j0, j1);
  return fm_after_launch() ? FASTMAX_ERR_LAUNCH : FASTMAX_OK;
}

inline int fm_maxnorm_dispatch(const FastmaxNormDesc* d0, const void* x0, void* keys0, const FastmaxNormDesc* d1,
                               const void* x1, void* keys1, fm_stream_t stream) {
  if (d0->dtype == FASTMAX_BF16)
    return d0->d == 64 ? fm_maxnorm_run<fm_bf16, 64>(d0, x0, keys0, d1, x1, keys1, stream)
                       : fm_maxnorm_run<fm_bf16, 32>(d0, x0, keys0, d1, x1, keys1, stream);
  return d0->d == 64 ? fm_maxnorm_run<float, 64>(d0, x0, keys0, d1, x1, keys1, stream)
                     : fm_maxnorm_run<float, 32>(d0, x0, keys0, d1, x1, keys1, stream);
}
