// Incremental decoding on a persistent moment state: what makes Fastmax generation O(1) per token.
//
// The causal kernel of the reference keeps running sums over the keys and adds one key per query
// (fastmax_cuda_forward.cu:160-276: the first nk - nq keys are summed before the first query, then one
// more per query).  Kept between calls, those sums are the whole memory of the sequence: a decoding step
// adds the new token's key and value to them and reads them out with the new query, without touching any
// earlier key (the reference's generation loop, transformer/eval.py:8-32, runs the whole context through the
// model for every new token).
//
// State of one batch*head, fp32, with k' = k * inv_tau and R = 1 + D (+ D*D for order 2) moment rows:
//     num [R][D]   row 0: sum v        rows 1 + m: sum k'_m v        rows 1 + D + m*D + l: sum k'_m k'_l v
//     den [R]      the same sums with v replaced by 1 (row 0: the number of keys)
// Readout for a query q:  F = a0 num[0] + a1 sum_m q_m num[1+m] + a2 sum_{m,l} q_m q_l num[1+D+mD+l],
// g likewise from den, o = F / g.
//
// k_decode_absorb: grid (ceil(R / 64), bh), 256 threads.  A workgroup owns 64 moment rows; a thread keeps four
// consecutive columns of FM_DEC_ROWS * D / 1024 of them in registers (16-byte loads and stores: D / 4 threads per
// row), adds the new tokens one after the other (their k', v staged through LDS), writes the rows back and, when
// a query is given (one new token), leaves its part of F and g in `part` [bh][blocks][D + 1]; k_decode_finish adds
// the parts in a fixed order and divides.  Bandwidth bound: a step reads and writes the state once (a thousand
// workgroups at the long shape's 16 heads; 256-row workgroups with one column per thread were a quarter as many and
// took 30 us for the 36 MB of a step).
#pragma once
#include "fm_kernels.h"

static constexpr int FM_DEC_ROWS = 64;      // moment rows per workgroup
constexpr int64_t fm_decode_rows(int d, bool quad) { return 1 + int64_t(d) + (quad ? int64_t(d) * d : 0); }
constexpr int fm_decode_blocks(int d, bool quad) { return int((fm_decode_rows(d, quad) + FM_DEC_ROWS - 1) / FM_DEC_ROWS); }
// floats of one batch*head's state: num [R][D] then den [R], R rounded up to whole blocks
inline int64_t fm_decode_state_floats(int d, bool quad) {
  return int64_t(fm_decode_blocks(d, quad)) * FM_DEC_ROWS * (d + 1);
}

// the two key features a moment row multiplies (index DH stands for the constant 1)
template <int DH> FM_DEVICE void fm_decode_row(int r, bool quad, int& m, int& l, bool& live) {
  live = true;
  if (r == 0) { m = DH; l = DH; }
  else if (r <= DH) { m = r - 1; l = DH; }
  else if (quad && r < 1 + DH + DH * DH) { m = (r - 1 - DH) / DH; l = (r - 1 - DH) % DH; }
  else { m = DH; l = DH; live = false; }
}

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS)
k_decode_absorb(TRef<const TIO> k, TRef<const TIO> v, TRef<const TIO> q, int n_new, int quad, float inv_tau, float a0,
                float a1, float a2, float* FM_RESTRICT state, float* FM_RESTRICT part) {
  constexpr int TPR = DH / 4;                            // threads per row (four columns each)
  constexpr int RPP = FM_THREADS / TPR;                  // rows per pass of the workgroup
  constexpr int RPT = FM_DEC_ROWS / RPP;                 // rows per thread
  constexpr int TB = 16;                                 // new tokens staged at a time
  static_assert(FM_DEC_ROWS % RPP == 0 && FM_DEC_ROWS <= FM_THREADS, "whole passes; one thread per denominator row");
  FM_SHARED float ks[TB][DH + 1];                        // k' of the staged tokens, [DH] = 1
  FM_SHARED __attribute__((aligned(16))) float vs[TB][DH];
  FM_SHARED float qs[DH + 1];
  FM_SHARED __attribute__((aligned(16))) float red[RPP][DH];
  FM_SHARED float redg[FM_THREADS / 64];
  const int tid = FM_TID_X, lane = tid & 63, bh = FM_BID_Y, blk = FM_BID_X;
  const int c4 = (tid % TPR) * 4, rsub = tid / TPR;
  const int64_t R = int64_t(FM_GDIM_X) * FM_DEC_ROWS;
  float* num = state + int64_t(bh) * R * (DH + 1);
  float* den = num + R * DH;
  const int r0 = blk * FM_DEC_ROWS;
  // this thread's rows (r0 + rsub + RPP * i), four columns of each, and their feature pairs
  fm_f32x4 acc[RPT];
  int rm[RPT], rl[RPT];
  bool rlive[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = r0 + rsub + RPP * i;
    acc[i] = *reinterpret_cast<const fm_f32x4*>(num + int64_t(r) * DH + c4);
    fm_decode_row<DH>(r, quad != 0, rm[i], rl[i], rlive[i]);
  }
  // denominators: thread t < FM_DEC_ROWS owns row r0 + t
  const bool down = tid < FM_DEC_ROWS;
  float dsum = down ? den[r0 + tid] : 0.f;
  int dm = DH, dl = DH; bool dlive = false;
  if (down) fm_decode_row<DH>(r0 + tid, quad != 0, dm, dl, dlive);
  for (int t0 = 0; t0 < n_new; t0 += TB) {
    FM_SYNC();
    for (int i = tid; i < TB * (DH + 1); i += FM_THREADS) {
      const int t = i / (DH + 1), f = i % (DH + 1);
      float x = 0.f;
      if (t0 + t < n_new) x = f < DH ? IO<TIO>::ld(k.base(bh) + int64_t(t0 + t) * k.s_n + f) * inv_tau : 1.0f;
      ks[t][f] = x;
    }
    for (int i = tid; i < TB * DH; i += FM_THREADS) {
      const int t = i / DH, f = i % DH;
      vs[t][f] = (t0 + t < n_new) ? IO<TIO>::ld(v.base(bh) + int64_t(t0 + t) * v.s_n + f) : 0.f;
    }
    FM_SYNC();
    const int nt = n_new - t0 < TB ? n_new - t0 : TB;
    for (int t = 0; t < nt; ++t) {
      const fm_f32x4 vc = *reinterpret_cast<const fm_f32x4*>(&vs[t][c4]);
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        const float w = rlive[i] ? ks[t][rm[i]] * ks[t][rl[i]] : 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += w * vc[j];
      }
      if (dlive) dsum += ks[t][dm] * ks[t][dl];
    }
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i)
    *reinterpret_cast<fm_f32x4*>(num + int64_t(r0 + rsub + RPP * i) * DH + c4) = acc[i];
  if (down) den[r0 + tid] = dsum;
  if (!part) return;
  // readout of the new token's query against the rows of this block
  FM_SYNC();
  if (tid <= DH) qs[tid] = tid < DH ? IO<TIO>::ld(q.base(bh) + tid) : 1.0f;
  FM_SYNC();
  fm_f32x4 f = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = r0 + rsub + RPP * i;
    const float coef = r == 0 ? a0 : (r <= DH ? a1 : a2);
    const float w = rlive[i] ? coef * qs[rm[i]] * qs[rl[i]] : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] += w * acc[i][j];
  }
  float gsum = dlive ? (r0 + tid == 0 ? a0 : (r0 + tid <= DH ? a1 : a2)) * qs[dm] * qs[dl] * dsum : 0.f;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) gsum += fm_shfl_xor(gsum, m);
  *reinterpret_cast<fm_f32x4*>(&red[rsub][c4]) = f;
  if (lane == 0) redg[tid >> 6] = gsum;
  FM_SYNC();
  if (tid < DH) {
    // the row groups in a fixed order
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < RPP; ++r) sum += red[r][tid];
    part[(int64_t(bh) * FM_GDIM_X + blk) * (DH + 1) + tid] = sum;
  } else if (tid == DH) {
    float gs = 0.f;
#pragma unroll
    for (int w = 0; w < FM_THREADS / 64; ++w) gs += redg[w];
    part[(int64_t(bh) * FM_GDIM_X + blk) * (DH + 1) + DH] = gs;
  }
}

// o = F / g from the parts of k_decode_absorb.  grid (bh), 256 threads: every wavefront adds a quarter of the
// blocks' parts, in order, and the four sums are added in a fixed order.
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS) k_decode_finish(const float* FM_RESTRICT part, int nblk, TRef<TIO> o, TRef<float> g) {
  FM_SHARED float red[FM_THREADS / 64][DH + 1];
  const int bh = FM_BID_X, tid = FM_TID_X, lane = tid & 63, wave = tid >> 6;
  const float* p = part + int64_t(bh) * nblk * (DH + 1);
  float f = 0.f, f2 = 0.f;
  const int per = (nblk + FM_THREADS / 64 - 1) / (FM_THREADS / 64), b0 = wave * per, b1 = b0 + per < nblk ? b0 + per : nblk;
  // all loads of the wavefront's blocks are issued before the first sum (a loop over a run-time count waits for
  // every load in turn: 17 memory latencies for the 66 blocks of D = 64, order 2)
  constexpr int PER_MAX = (fm_decode_blocks(DH, true) + FM_THREADS / 64 - 1) / (FM_THREADS / 64);
  const bool gl = DH == 64 ? lane == 0 : lane == DH;     // the lane that also adds the g parts
  float x[PER_MAX], x2[PER_MAX];
#pragma unroll
  for (int i = 0; i < PER_MAX; ++i) {
    const int b = b0 + i;
    x[i] = (b < b1 && lane < DH) ? p[b * (DH + 1) + lane] : 0.f;
    x2[i] = (b < b1 && gl) ? p[b * (DH + 1) + DH] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < PER_MAX; ++i) { f += x[i]; f2 += x2[i]; }
  if (lane < DH) red[wave][lane] = f;
  if (DH == 64 ? lane == 0 : lane == DH) red[wave][DH] = f2;
  FM_SYNC();
  if (tid <= DH) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < FM_THREADS / 64; ++w) sum += red[w][tid];
    red[0][tid] = sum;
  }
  FM_SYNC();
  const float gs = red[0][DH];
  if (tid < DH) IO<TIO>::st(o.base(bh) + tid, red[0][tid] / gs);
  if (tid == 0) g.base(bh)[0] = gs;
}

template <typename TIO, int DH>
int fm_decode_run(const FastmaxDesc* d, const void* q, const void* k, const void* v, int n_new, float* state, void* o,
                  float* g, float* scratch, fm_stream_t stream) {
  const bool quad = d->p == 2 && d->a2 != 0.0f;
  const int nblk = fm_decode_blocks(DH, quad);
  const TRef<const TIO> kr = fm_ref<const TIO>(static_cast<const TIO*>(k), d->sk), vr = fm_ref<const TIO>(static_cast<const TIO*>(v), d->sv);
  const TRef<const TIO> qr = q ? fm_ref<const TIO>(static_cast<const TIO*>(q), d->sq) : kr;
  FM_KERNEL_LAUNCH((k_decode_absorb<TIO, DH>), fm_dim3(nblk, d->bh), fm_dim3(FM_THREADS), 0, stream, kr, vr, qr, n_new, quad ? 1 : 0,
                   d->inv_tau, d->a0, d->a1, quad ? d->a2 : 0.0f, state, q ? scratch : nullptr);
  if (q)
    FM_KERNEL_LAUNCH((k_decode_finish<TIO, DH>), fm_dim3(d->bh), fm_dim3(FM_THREADS), 0, stream, scratch, nblk,
                     fm_ref<TIO>(static_cast<TIO*>(o), d->so), fm_ref<float>(g, d->sg));
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
