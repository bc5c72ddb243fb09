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
//
// k_decode_absorb_mma (further down): the same sums for a whole prompt with matrix instructions, one launch.
#pragma once
#include "fm_kernels.h"

static constexpr int FM_DEC_ROWS = 64;      // the moment rows of a state are padded to a multiple of this
static constexpr int FM_DEC_THREADS = 512;  // eight wavefronts per workgroup: five rows per thread at D = 64, order 2 (per token: 256 threads 9.3 us, 384 7.7, 512 and 768 7.4, 1024 7.7)
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
  if (has_q && tid <= DH) qs[tid] = qreg;             // read after the barriers of the token loop
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
  // same sum), then the wavefronts in order
  if (n_new <= 0) FM_SYNC();                           // (no token: qs has not met a barrier yet)
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
  if (tid < 4) {
    // each of the four output threads adds its column and the denominator itself (one barrier less than a shared sum)
    float sum = 0.f, gs = 0.f;
#pragma unroll
    for (int w = 0; w < FM_DEC_THREADS / 64; ++w) { sum += red[w][tid]; gs += red[w][4]; }
    IO<TIO>::st(o.base(bh) + c4 + tid, sum / gs);
    if (tid == 0 && cb == 0) g.base(bh)[0] = gs;
  }
}

// ------------------------------------------------------------------------------
// k_decode_absorb_mma: a prompt's keys and values added to the state with matrix instructions (bf16 tensors, D = 64,
// order 2).  k_decode adds tokens one after the other on the vector units: 2 145 rows x 4 columns of multiply-adds
// per token and workgroup, 1.7 ms for 4 096 tokens at 16 batch*heads; the same sums are three 32 x 32 x 16 products
// per 16 tokens and value column.
//
// grid (D / 4, bh), 256 threads: the workgroup owns the same [R][4] block of the state as in k_decode, wavefront w its
// value column c = 4 cb + w.  Per tile of 128 tokens the keys (times inv_tau, as _Float16) are staged row-major and
// the four value columns, a row of ones (zero past the end of the prompt) and three rows of zeros as rows over the
// tokens.  Per k-step of 16 tokens a wavefront reads the two key fragments with transposing LDS reads and uses them
// as B operand and, times its value column's fragment, as A operand: the slice  sum_t v_tc k'_ta k'_tb  of its column
// on the three 32 x 32 tiles on and above the diagonal (it is symmetric in a, b), as k_walk_sym does.  What all four
// columns share is dealt by k-step, wavefront w taking the k-steps u = w (mod 4): the denominators' order-2 sums
// (the same three products with the bare key fragments), and the rows 0 .. D of numerators and denominators in one go
// as  sum_t z_tn' x_tn  with z = (k', then the rows of x) and x = (the four value columns, ones, zeros): three more
// products.  At the end the four wavefronts' parts of the shared sums meet in LDS and are added in a fixed order, and
// every sum is ADDED to the state in memory (each address by exactly one lane: no atomics, the same bits every run).
// Operands are rounded to _Float16 (k', and the products v k'), the sums are fp32.
template <int DH> struct DecAbsCfg {
  typedef Mma<fm_half> M;
  static constexpr int TT = 128;                       // tokens per tile
  static constexpr int PQ = DH + M::PAD;               // pitch of the key rows
  static constexpr int XR = 8;                         // rows over tokens: four value columns, ones, three of zeros
  static constexpr int XP = TT + M::PAD;
  static constexpr int TILE_E = TT * PQ + XR * XP;
  static constexpr int NSH = 6;                        // accumulator tiles of the shared sums per wavefront
  static constexpr size_t RED_BYTES = size_t(4) * (NSH / 2) * 16 * 64 * 4;   // they meet in LDS three tiles at a time
  static constexpr size_t lds_bytes() { return size_t(2) * TILE_E * 2 > RED_BYTES ? size_t(2) * TILE_E * 2 : RED_BYTES; }
};

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, 1)
k_decode_absorb_mma(TRef<const TIO> k, TRef<const TIO> v, int n_new, float inv_tau, float* FM_RESTRICT state) {
  static_assert(DH == 64, "two 32-row tiles per feature axis");
  typedef fm_half E;
  typedef Mma<E> M;
  typedef typename M::frag frag;
  typedef DecAbsCfg<DH> C;
  constexpr int TT = C::TT, PQ = C::PQ, XP = C::XP, NSTEP = TT / M::KSTEP;
  FM_DYN_SMEM(smem);
  E* const buf0 = reinterpret_cast<E*>(smem);
  E* const buf1 = buf0 + C::TILE_E;
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  // the sixteen workgroups of a batch*head read the same keys: behind one L2 (145 -> 28 MB fetched for 4 096 tokens at 16 heads, 0.125 -> 0.097 ms)
  int cb, bh;
  fm_xcd_map(FM_GDIM_X, FM_GDIM_Y, cb, bh);
  const int c4 = 4 * cb;
  const int64_t Rp = fm_decode_rows_padded(DH, true);
  float* num = state + (int64_t(bh) * (DH / 4) + cb) * Rp * 5;
  float* den = num + Rp * 4;
  const TIO* kb = k.base(bh);
  const TIO* vb = v.base(bh);

  // global memory -> registers: a thread's four 16-byte pieces of the key rows, and (threads below TT) a token's four values
  constexpr int CPR = DH / 8, NK = TT * CPR / FM_THREADS;
  float kreg[NK][8], vreg[4];
  auto fetch = [&](int t0) FM_ALWAYS_INLINE {
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      const int c = tid + FM_THREADS * i, row = t0 + c / CPR, f0 = (c % CPR) * 8;
      if (row < n_new) IO<TIO>::ld8(kb + int64_t(row) * k.s_n + f0, k.vec != 0, kreg[i]);
      else {
#pragma unroll
        for (int j = 0; j < 8; ++j) kreg[i][j] = 0.f;
      }
    }
    if (tid < TT) {
#pragma unroll
      for (int j = 0; j < 4; ++j) vreg[j] = (t0 + tid < n_new) ? IO<TIO>::ld(vb + int64_t(t0 + tid) * v.s_n + c4 + j) : 0.f;
    }
  };
  auto put = [&](E* b, int t0) FM_ALWAYS_INLINE {
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      const int c = tid + FM_THREADS * i;
      float sc[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) sc[j] = kreg[i][j] * inv_tau;
      CE<E>::st8(b + (c / CPR) * PQ + (c % CPR) * 8, sc);
    }
    if (tid < TT) {
      E* x = b + TT * PQ + tid;
#pragma unroll
      for (int j = 0; j < 4; ++j) x[j * XP] = E(vreg[j]);
      x[4 * XP] = E(t0 + tid < n_new ? 1.0f : 0.0f);
    }
  };
  // rows 5 .. 7 of both buffers: zeros, written once
  for (int i = tid; i < 2 * 3 * XP; i += FM_THREADS) {
    E* b = i < 3 * XP ? buf0 : buf1;
    b[TT * PQ + 5 * XP + (i % (3 * XP))] = E(0.0f);
  }

  fm_f32x16 a00 = fm_zero16(), a01 = fm_zero16(), a11 = fm_zero16();       // the wavefront's value column
  fm_f32x16 sh[C::NSH];                                                     // its part of the shared sums: d00, d01, d11, l0, l1, r0
#pragma unroll
  for (int i = 0; i < C::NSH; ++i) sh[i] = fm_zero16();

  fetch(0);
  put(buf0, 0);
  if (TT < n_new) fetch(TT);
  FM_SYNC();
  int par = 0;
  for (int t0 = 0; t0 < n_new; t0 += TT) {
    const E* cbuf = par ? buf1 : buf0;
    const E* xt = cbuf + TT * PQ;
#pragma unroll
    for (int u = 0; u < NSTEP; ++u) {
      const frag k0 = M::load_tr(cbuf, PQ, 16 * u, 0, lane), k1 = M::load_tr(cbuf, PQ, 16 * u, 32, lane);
      const frag xv = M::load_nat_perm(xt + wave * XP, u, lh);
      const frag f0 = k0 * xv, f1 = k1 * xv;
      a00 = M::mma(f0, k0, a00);
      a01 = M::mma(f0, k1, a01);
      a11 = M::mma(f1, k1, a11);
      if ((u & 3) == wave) {
        const frag xs = M::load_nat_perm(xt + (lr < C::XR ? lr : C::XR - 1) * XP, u, lh);   // rows past the eighth: zeros
        sh[0] = M::mma(k0, k0, sh[0]);
        sh[1] = M::mma(k0, k1, sh[1]);
        sh[2] = M::mma(k1, k1, sh[2]);
        sh[3] = M::mma(k0, xs, sh[3]);
        sh[4] = M::mma(k1, xs, sh[4]);
        sh[5] = M::mma(xs, xs, sh[5]);
      }
    }
    if (t0 + TT < n_new) {
      put(par ? buf0 : buf1, t0 + TT);
      if (t0 + 2 * TT < n_new) fetch(t0 + 2 * TT);
    }
    FM_SYNC();
    par ^= 1;
  }

  // the wavefront's own column: entries (a, b) with a <= b go to their pair rows
  auto pair_row = [&](int a, int b) { return 1 + DH + a * DH - a * (a - 1) / 2 + (b - a); };
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int ra = fm_acc_row(e, lh);
    if (ra <= lr) num[int64_t(pair_row(ra, lr)) * 4 + wave] += a00[e];
    num[int64_t(pair_row(ra, 32 + lr)) * 4 + wave] += a01[e];
    if (ra <= lr) num[int64_t(pair_row(32 + ra, 32 + lr)) * 4 + wave] += a11[e];
  }
  // the shared sums: the four parts through LDS (the staging buffers are spent: the loop ended on a barrier), three
  // tiles at a time; wavefront w adds entries 4 w .. 4 w + 3 of every tile in the order of the wavefronts
  float* red = reinterpret_cast<float*>(smem);           // [wave][tile of the round][e][lane]
  constexpr int HALF = C::NSH / 2;
#pragma unroll
  for (int rnd = 0; rnd < 2; ++rnd) {
    if (rnd) FM_SYNC();
#pragma unroll
    for (int i = 0; i < HALF; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) red[((wave * HALF + i) * 16 + e) * 64 + lane] = sh[rnd * HALF + i][e];
    FM_SYNC();
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
#pragma unroll
      for (int e4 = 0; e4 < 4; ++e4) {
        const int e = 4 * wave + e4;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) sum += red[((w * HALF + i) * 16 + e) * 64 + lane];
        const int ra = fm_acc_row(e, lh);
        if (rnd == 0) {
          // denominators of the pair rows: tiles (0,0), (0,1), (1,1)
          if (i == 0) { if (ra <= lr) den[pair_row(ra, lr)] += sum; }
          else if (i == 1) den[pair_row(ra, 32 + lr)] += sum;
          else if (ra <= lr) den[pair_row(32 + ra, 32 + lr)] += sum;
        } else if (i < 2) {
          // rows 1 + a: column n < 4 a numerator, n = 4 the denominator
          const int a = 32 * i + ra;
          if (lr < 4) num[int64_t(1 + a) * 4 + lr] += sum;
          else if (lr == 4) den[1 + a] += sum;
        } else if (ra == 4) {
          // row 0: the ones row of z against the columns of x
          if (lr < 4) num[lr] += sum;
          else if (lr == 4) den[0] += sum;
        }
      }
    }
  }
}

// prompts of bf16 tensors at D = 64, order 2, from this many tokens on go through k_decode_absorb_mma (below it the
// one launch of k_decode is as quick, and it keeps fp32 products)
static constexpr int FM_DEC_MMA_MIN = 64;
template <typename TIO, int DH> inline bool fm_decode_absorb_mma_applies(bool quad, bool has_q, int n_new) {
  return sizeof(TIO) == 2 && DH == 64 && quad && !has_q && n_new >= FM_DEC_MMA_MIN;
}

template <typename TIO, int DH>
int fm_decode_run(const FastmaxDesc* d, const void* q, const void* k, const void* v, int n_new, float* state, void* o,
                  float* g, float* scratch, fm_stream_t stream) {
  const bool quad = d->p == 2 && d->a2 != 0.0f;
  const int nblk = fm_decode_blocks(DH, quad);
  const TRef<const TIO> kr = fm_ref<const TIO>(static_cast<const TIO*>(k), d->sk), vr = fm_ref<const TIO>(static_cast<const TIO*>(v), d->sv);
  const TRef<const TIO> qr = q ? fm_ref<const TIO>(static_cast<const TIO*>(q), d->sq) : kr;
  (void)scratch; (void)nblk;
  if constexpr (sizeof(TIO) == 2 && DH == 64) {
    if (fm_decode_absorb_mma_applies<TIO, DH>(quad, q != nullptr, n_new)) {
      typedef DecAbsCfg<DH> C;
      FM_KERNEL_LAUNCH((k_decode_absorb_mma<TIO, DH>), fm_dim3(DH / 4, d->bh), fm_dim3(FM_THREADS), C::lds_bytes(), stream, kr, vr,
                       n_new, d->inv_tau, state);
      return fm_after_launch() ? FASTMAX_ERR_LAUNCH : FASTMAX_OK;
    }
  }
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
