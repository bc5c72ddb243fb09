// Incremental decoding on a persistent moment state: what makes Fastmax generation O(1) per token.
//
// The causal kernel of the reference keeps running sums over the keys and adds one key per query
// (fastmax_cuda_forward.cu:160-276: the first nk - nq keys are summed before the first query, then one
// more per query).  Kept between calls, those sums are the whole memory of the sequence: a decoding step
// adds the new token's key and value to them and reads them out with the new query, without touching any
// earlier key (the reference's generation loop, transformer/eval.py:8-32, runs the whole context through the
// model for every new token).
//
// State of one batch*head, fp32, with k' = k * inv_tau and R = 1 + D (+ D (D + 1) / 2 for order 2) moment rows:
//     num [R][D]   row 0: sum v        rows 1 + m: sum k'_m v        rows 1 + D + pair(m, l): sum k'_m k'_l v,  m <= l
//     den [R]      the same sums with v replaced by 1 (row 0: the number of keys)
// The order-2 sums are symmetric in (m, l), so only the pairs m <= l are kept (2 080 of 4 096 rows at D = 64: a step
// reads and writes the state once, and this halves it), in row-major order of the upper triangle.
// Readout for a query q:  F = a0 num[0] + a1 sum_m q_m num[1+m] + a2 sum_{m<=l} w_ml q_m q_l num[1+D+pair(m,l)] with
// w_ml = 1 on the diagonal and 2 off it; g likewise from den, o = F / g.
//
// k_decode: grid (D / 4, bh), 512 threads, ONE launch per step.  A workgroup owns four value columns of every moment
// row (a contiguous [R][4] block of the state, 16-byte loads and stores) and a copy of the denominator column, so the
// sums over the rows that the readout needs (F of its four columns, and g) never leave the workgroup: no partial
// results in memory, no second launch, no fence.  A thread keeps its rows (every 512th) in registers, adds the new
// tokens one after the other (their k' and the four v columns staged through LDS), writes the rows back and, when a
// query is given (one new token), the workgroup adds up its part of the readout in a fixed order and stores its four
// outputs.  Bandwidth and latency bound: a step reads and writes the state once (the denominators once per
// workgroup: 5 floats per row and workgroup instead of 4).
#pragma once
#include "fm_kernels.h"

static constexpr int FM_DEC_ROWS = 64;      // the moment rows of a state are padded to a multiple of this
static constexpr int FM_DEC_THREADS = 512;  // eight wavefronts per workgroup: five rows per thread at D = 64, order 2 (256: 9.3 us per token, 1024: 7.9)
constexpr int64_t fm_decode_rows(int d, bool quad) { return 1 + int64_t(d) + (quad ? int64_t(d) * (d + 1) / 2 : 0); }
constexpr int fm_decode_blocks(int d, bool quad) { return int((fm_decode_rows(d, quad) + FM_DEC_ROWS - 1) / FM_DEC_ROWS); }
// floats of one batch*head's state: per group of four value columns num [Rp][4] then den [Rp], Rp = R rounded up to whole blocks
constexpr int64_t fm_decode_rows_padded(int d, bool quad) { return int64_t(fm_decode_blocks(d, quad)) * FM_DEC_ROWS; }
inline int64_t fm_decode_state_floats(int d, bool quad) { return fm_decode_rows_padded(d, quad) * 5 * (d / 4); }

// the two key features a moment row multiplies (index DH stands for the constant 1) and how often the row counts in
// a readout (an order-2 row off the diagonal stands for the pairs (m, l) and (l, m))
template <int DH> FM_DEVICE void fm_decode_row(int r, bool quad, int& m, int& l, bool& live, float& mult) {
  live = true; mult = 1.0f;
  if (r == 0) { m = DH; l = DH; }
  else if (r <= DH) { m = r - 1; l = DH; }
  else if (quad && r < 1 + DH + DH * (DH + 1) / 2) {
    // pair index p -> (m, l), m <= l, rows of the upper triangle one after the other: row m starts at m D - m (m - 1) / 2
    // (m from the root of the quadratic, then one step either way against rounding)
    const int p = r - 1 - DH;
    m = int(0.5f * (float(2 * DH + 1) - fm_sqrtf(float((2 * DH + 1) * (2 * DH + 1) - 8 * p))));
    if (m < 0) m = 0;
    if (m > DH - 1) m = DH - 1;
    if (m * DH - m * (m - 1) / 2 > p) --m;
    else if (m + 1 < DH && (m + 1) * DH - (m + 1) * m / 2 <= p) ++m;
    l = m + (p - (m * DH - m * (m - 1) / 2));
    if (l != m) mult = 2.0f;
  } else { m = DH; l = DH; live = false; }
}

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_DEC_THREADS)
k_decode(TRef<const TIO> k, TRef<const TIO> v, TRef<const TIO> q, int n_new, int quad, float inv_tau, float a0,
         float a1, float a2, float* FM_RESTRICT state, TRef<TIO> o, TRef<float> g, int has_q) {
  constexpr int TB = 16;                                 // new tokens staged at a time
  constexpr int NI = (int(fm_decode_rows(DH, true)) + FM_DEC_THREADS - 1) / FM_DEC_THREADS;   // rows per thread at most
  FM_SHARED float ks[TB][DH + 1];                        // k' of the staged tokens, [DH] = 1
  FM_SHARED __attribute__((aligned(16))) float vs[TB][4];
  FM_SHARED float qs[DH + 1];
  FM_SHARED float red[FM_DEC_THREADS / 64][5];
  const int tid = FM_TID_X, cb = FM_BID_X, bh = FM_BID_Y, c4 = 4 * cb;
  const int R = int(fm_decode_rows(DH, quad != 0));
  const int64_t Rp = fm_decode_rows_padded(DH, quad != 0);
  float* num = state + (int64_t(bh) * (DH / 4) + cb) * Rp * 5;
  float* den = num + Rp * 4;
  fm_f32x4 acc[NI];
  float dsum[NI], rmult[NI];
  int rm[NI], rl[NI];
  bool rlive[NI];
  // the query travels with the state's rows (one memory latency for both)
  float qreg = 1.0f;
  if (has_q && tid < DH) qreg = IO<TIO>::ld(q.base(bh) + tid);
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int r = tid + FM_DEC_THREADS * i;
    rlive[i] = false; rm[i] = DH; rl[i] = DH; rmult[i] = 1.0f; dsum[i] = 0.f;
    acc[i] = fm_f32x4{0.f, 0.f, 0.f, 0.f};
    if (r < R) {
      acc[i] = *reinterpret_cast<const fm_f32x4*>(num + int64_t(r) * 4);
      dsum[i] = den[r];
      fm_decode_row<DH>(r, quad != 0, rm[i], rl[i], rlive[i], rmult[i]);
    }
  }
  for (int t0 = 0; t0 < n_new; t0 += TB) {
    FM_SYNC();
    for (int i = tid; i < TB * (DH + 1); i += FM_DEC_THREADS) {
      const int t = i / (DH + 1), f = i % (DH + 1);
      float x = 0.f;
      if (t0 + t < n_new) x = f < DH ? IO<TIO>::ld(k.base(bh) + int64_t(t0 + t) * k.s_n + f) * inv_tau : 1.0f;
      ks[t][f] = x;
    }
    if (tid < TB * 4) {
      const int t = tid / 4, f = tid % 4;
      vs[t][f] = (t0 + t < n_new) ? IO<TIO>::ld(v.base(bh) + int64_t(t0 + t) * v.s_n + c4 + f) : 0.f;
    }
    FM_SYNC();
    const int nt = n_new - t0 < TB ? n_new - t0 : TB;
    for (int t = 0; t < nt; ++t) {
      const fm_f32x4 vc = *reinterpret_cast<const fm_f32x4*>(&vs[t][0]);
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const float w = rlive[i] ? ks[t][rm[i]] * ks[t][rl[i]] : 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += w * vc[j];
        dsum[i] += w;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int r = tid + FM_DEC_THREADS * i;
    if (r < R) {
      *reinterpret_cast<fm_f32x4*>(num + int64_t(r) * 4) = acc[i];
      den[r] = dsum[i];
    }
  }
  if (!has_q) return;
  // readout of the new token's query: the thread's rows, then the wavefront (a butterfly: every lane ends with the
  // same sum), then the four wavefronts in order
  if (tid <= DH) qs[tid] = qreg;
  FM_SYNC();
  float f[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int r = tid + FM_DEC_THREADS * i;
    const float coef = r == 0 ? a0 : (r <= DH ? a1 : a2);
    const float w = rlive[i] ? coef * rmult[i] * qs[rm[i]] * qs[rl[i]] : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] += w * acc[i][j];
    f[4] += w * dsum[i];
  }
#pragma unroll
  for (int j = 0; j < 5; ++j) {
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) f[j] += fm_shfl_xor(f[j], m);
  }
  if ((tid & 63) == 0) {
#pragma unroll
    for (int j = 0; j < 5; ++j) red[tid >> 6][j] = f[j];
  }
  FM_SYNC();
  if (tid < 5) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < FM_DEC_THREADS / 64; ++w) sum += red[w][tid];
    red[0][tid] = sum;
  }
  FM_SYNC();
  const float gs = red[0][4];
  if (tid < 4) IO<TIO>::st(o.base(bh) + c4 + tid, red[0][tid] / gs);
  if (tid == 0 && cb == 0) g.base(bh)[0] = gs;
}

template <typename TIO, int DH>
int fm_decode_run(const FastmaxDesc* d, const void* q, const void* k, const void* v, int n_new, float* state, void* o,
                  float* g, float* scratch, fm_stream_t stream) {
  const bool quad = d->p == 2 && d->a2 != 0.0f;
  const int nblk = fm_decode_blocks(DH, quad);
  const TRef<const TIO> kr = fm_ref<const TIO>(static_cast<const TIO*>(k), d->sk), vr = fm_ref<const TIO>(static_cast<const TIO*>(v), d->sv);
  const TRef<const TIO> qr = q ? fm_ref<const TIO>(static_cast<const TIO*>(q), d->sq) : kr;
  (void)scratch; (void)nblk;
  const TRef<TIO> orf = q ? fm_ref<TIO>(static_cast<TIO*>(o), d->so) : TRef<TIO>{nullptr, 0, 0, 0, 0, 0};
  const TRef<float> grf = q ? fm_ref<float>(g, d->sg) : TRef<float>{nullptr, 0, 0, 0, 0, 0};
  FM_KERNEL_LAUNCH((k_decode<TIO, DH>), fm_dim3(DH / 4, d->bh), fm_dim3(FM_DEC_THREADS), 0, stream, kr, vr, qr, n_new, quad ? 1 : 0,
                   d->inv_tau, d->a0, d->a1, quad ? d->a2 : 0.0f, state, orf, grf, q ? 1 : 0);
  return fm_after_launch() ? FASTMAX_ERR_LAUNCH : FASTMAX_OK;
}

inline int fm_decode_dispatch(const FastmaxDesc* d, const void* q, const void* k, const void* v, int n_new, float* state,
                              void* o, float* g, float* scratch, fm_stream_t stream) {
  if (d->dtype == FASTMAX_BF16)
    return d->d == 64 ? fm_decode_run<fm_bf16, 64>(d, q, k, v, n_new, state, o, g, scratch, stream)
                      : fm_decode_run<fm_bf16, 32>(d, q, k, v, n_new, state, o, g, scratch, stream);
  return d->d == 64 ? fm_decode_run<float, 64>(d, q, k, v, n_new, state, o, g, scratch, stream)
                    : fm_decode_run<float, 32>(d, q, k, v, n_new, state, o, g, scratch, stream);
}
