// Order 1 on long sequences (bf16 tensors, _Float16 arithmetic, causal, 128-token segments): a path of its
// own that reads the caller's tensors directly and is bound by the bytes it moves.
//
// With f(s) = a0 + a1 s every term that crosses a segment boundary is a D x D sum, and the score gradient
// does not depend on the score, dS_ij = a1 (gh_i.v_j - c_i):
//     F_i   = a0 sum_{j<=i} v_j + a1 (sum_{j<=i} v_j k'_j^T) q'_i          g_i = a0 (i + 1) + a1 q'_i . sum_{j<=i} k'_j
//     dq'_i = a1 [ (sum_{j<=i} k'_j v_j^T) gh_i - c_i sum_{j<=i} k'_j ]
//     dk'_j = a1 [ (sum_{i>=j} q'_i gh_i^T) v_j - sum_{i>=j} c_i q'_i ]
//     dv_j  = a0 sum_{i>=j} gh_i + a1 (sum_{i>=j} gh_i q'_i^T) k'_j
// so a segment needs its own 128 rows, the sums over the segments before it (keys, values) and after it
// (queries, gh), and nothing else.  Four kernels:
//   k_o1_sums<KV>  k, v            -> one workgroup per run of segments: for every segment the sums over the segments
//                                     before it inside the run, and the run's total (k_o1_runscan: totals -> sums over
//                                     the runs before); a consumer adds the two parts
//   k_o1_fwd       q, k, v, prefix -> o, g            (one workgroup per segment)
//   k_o1_sums<QG>  q, dO, o, g     -> the same, walking backwards
//   k_o1_bwd       q, k, v, dO, o, g, prefix, suffix -> dq, dk, dv      (one workgroup per segment)
// No converted or transposed copy of any tensor is written: rows are converted (and scaled: 1/tau, the
// folded normalisation, the gradient scale) in registers on their way into LDS.  The general kernels need a
// conversion pass per tensor, read the four operand copies once per gradient and stream every tile of a
// segment again per 128 own tokens.  Replaces, for this case, calc_masked (fastmax_cuda_forward.cu:146-280)
// and calc_gradq/k/v_masked (fastmax_cuda_backward.cu:101-188, 272-358, 430-491).
#pragma once
#include "fm_tok.h"

static constexpr int FM_O1_SEG = 128;
static constexpr int FM_O1_DQ_PITCH = 40;   // elements per row of k_o1_bwd's per-wavefront output staging (32 features, rows 16-byte aligned)

// One 128-token segment of a bf16 caller tensor as raw 16-byte chunks: with CPR = DH / 8 chunks per row,
// thread t holds chunk t % CPR of the rows t / CPR + (256 / CPR) i.  Rows past the end are zeros.
template <int DH> struct O1Raw {
  static constexpr int CPR = DH / 8, N = FM_O1_SEG * CPR / FM_THREADS, RSTEP = FM_THREADS / CPR;
  fm_u32x4 r[N];
  FM_DEVICE void load(const TRef<const fm_bf16>& x, int bh, int t0, int n, int tid) {
    const fm_bf16* base = x.base(bh);
    const int col = (tid % CPR) * 8;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int row = t0 + tid / CPR + RSTEP * i;
      fm_u32x4 z = {0u, 0u, 0u, 0u};
      if (row < n) {
        const fm_bf16* p = base + int64_t(row) * x.s_n + col;
        if (x.vec) z = *reinterpret_cast<const fm_u32x4*>(p);
        else {
#pragma unroll
          for (int j = 0; j < 4; ++j) z[j] = uint32_t(p[2 * j]) | (uint32_t(p[2 * j + 1]) << 16);
        }
      }
      r[i] = z;
    }
  }
  // chunk i as eight floats
  FM_DEVICE void unpack(int i, float out[8]) const {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t lo = r[i][j] << 16, hi = r[i][j] & 0xffff0000u;
      __builtin_memcpy(&out[2 * j], &lo, 4);
      __builtin_memcpy(&out[2 * j + 1], &hi, 4);
    }
  }
  static FM_DEVICE int row_of(int i, int tid) { return tid / CPR + RSTEP * i; }     // inside the segment
  static FM_DEVICE int col_of(int tid) { return (tid % CPR) * 8; }
  // converted (times scale) into an LDS tile [128][pitch]
  FM_DEVICE void store(fm_half* lds, int pitch, int tid, float scale) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      float f[8];
      unpack(i, f);
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] *= scale;
      CE<fm_half>::st8(lds + row_of(i, tid) * pitch + col_of(tid), f);
    }
  }
};

// gh = gscale * dO / g and c = gh . o of the segment's rows, from raw dO and o chunks and the denominators gi of
// the thread's rows (1 past the end): gh rows go to the LDS
// tile Gs, c to cs (compute type, 16-token groups in `tperm` order: the weights of a matrix product) or to cf
// (fp32, natural order: what the score gradient subtracts), whichever is given.  Every lane takes part in the shuffles.
template <int DH>
FM_DEVICE void fm_o1_gh_rows(const O1Raw<DH>& rdo, const O1Raw<DH>& ro, const float* gi, float gscale, fm_half* Gs,
                             int pitch, fm_half* cs, float* cf, int tid) {
  typedef O1Raw<DH> R;
#pragma unroll
  for (int i = 0; i < R::N; ++i) {
    const int row = R::row_of(i, tid);
    const float ginv = gscale / gi[i];
    float a[8], b[8];
    rdo.unpack(i, a);
    ro.unpack(i, b);
    float csum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) { a[j] *= ginv; csum += a[j] * b[j]; }
#pragma unroll
    for (int m = 1; m < R::CPR; m <<= 1) csum += fm_shfl_xor(csum, m);
    CE<fm_half>::st8(Gs + row * pitch + R::col_of(tid), a);
    if (tid % R::CPR == 0) {
      if (cs) cs[Mma<fm_half>::tperm(row)] = CE<fm_half>::from(csum);
      if (cf) cf[row] = csum;
    }
  }
}

// ------------------------------------------------------------------------------
// k_o1_sums: the sums over a run of `run_len` consecutive segments, one workgroup per run.  grid (1, bh, runs).
// A prefix walk takes the run's segments in ascending order, a suffix walk in descending order; before a segment
// is added, the sums so far go to the segment's slot (the state of the segments before / after it INSIDE its
// run), and at the end the run's total goes to `runtot`.  k_o1_runscan then turns the totals into the sums over
// the runs before / after each run; a consumer adds the two.  (Per-segment sums followed by a scan over all
// segments moved every state three times more and ran the scan on a handful of wavefronts.)
//   QG = 0: operands p = v, r = k':   slab [r][c] = coef1 sum p_r r_c, va = coefva sum k', vb = coefvb sum v
//   QG = 1: operands p = q', r = gh:  the same slab, va = coefva sum c q', vb = coefvb sum gh
// The eight 32x32 tiles of the sums (D = 64) are dealt to the wavefronts, two each; the next segment's rows travel
// from global memory to registers while this one's products run.
// A run total (and `runtot` after the scan): DH * DH + 2 * DH floats, the slab, then va, then vb.
// ------------------------------------------------------------------------------
template <int DH> struct O1Run {
  static constexpr int RS = DH * DH + 2 * DH;      // floats of a run total
  static constexpr int VS = 2 * DH;                // floats of a segment's vector sums (`small`: [bh][segments][VS], va then vb)
};
// Segments per run: enough runs to give every CU two workgroups, runs as long as that allows (measured on
// MI355X, B*H = 16, 512 segments each: 16 segments per run 0.19 ms for both sums passes of a step, 8: 0.205,
// 32: 0.215, 64: 0.38).
inline int fm_o1_run_len(int nseg, int bh) {
  const int64_t r = int64_t(nseg) * bh / 512;
  return r < 2 ? 2 : (r > 32 ? 32 : int(r));
}
inline int fm_o1_runs(int nseg, int run_len) { return (nseg + run_len - 1) / run_len; }

template <typename TIO> struct O1SumArgs {
  TRef<const TIO> x0, x1;            // QG = 0: k, v          QG = 1: q, dO
  TRef<const TIO> o; TRef<const float> g;     // QG = 1
  float scale0;                      // on x0: sqrt(1/tau)
  NormFold fold0;                    // folded normalisation of x0
  const float* gpart; int gnblk;     // QG = 1: see k_grad_scale
  int n;
  BuildArgs<fm_half> b;              // where the segments' states go and their coefficients (big, small, nslots = nseg, mode, coef*)
  float* runtot;                     // [bh][runs][O1Run::RS]
  int run_len;                       // segments per run
};

template <typename TIO, int DH, int QG>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, 2) k_o1_sums(O1SumArgs<TIO> A) {
  typedef fm_half E;
  typedef Mma<E> M;
  typedef typename M::frag frag;
  typedef O1Raw<DH> R;
  constexpr int NT = DH / 32, NTILE = NT * NT + 2 * NT, NS = (NTILE + 3) / 4;
  constexpr int TT = FM_O1_SEG, PQ = DH + M::PAD;
  FM_DYN_SMEM(smem);
  E* Lp = reinterpret_cast<E*>(smem);                  // [TT][PQ] each
  E* Lr = Lp + TT * PQ;
  E* Lc = Lr + TT * PQ;                                // [TT] weights (QG)
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  const int bh = FM_BID_Y, run = FM_BID_Z, nruns = FM_GDIM_Z;
  const int s_lo = run * A.run_len, s_hi = s_lo + A.run_len < A.b.nseg ? s_lo + A.run_len : A.b.nseg;
  const int cnt = s_hi - s_lo;
  const bool suffix = A.b.mode == FM_WALK_SUFFIX;
  E* big = A.b.big + int64_t(bh) * A.b.nslots * StateDims<DH>::stride(false);
  float* sml = A.b.small + int64_t(bh) * A.b.nslots * O1Run<DH>::VS;
  R r0, r1, ro;
  float gi[R::N];
  auto fetch = [&](int seg) FM_ALWAYS_INLINE {
    const int tb = seg * TT;
    r0.load(A.x0, bh, tb, A.n, tid);
    r1.load(A.x1, bh, tb, A.n, tid);
    if (QG) {
      ro.load(A.o, bh, tb, A.n, tid);
#pragma unroll
      for (int i = 0; i < R::N; ++i) {
        const int row = tb + R::row_of(i, tid);
        gi[i] = row < A.n ? A.g.base(bh)[int64_t(row) * A.g.s_n] : 1.0f;
      }
    }
  };
  fetch(suffix ? s_hi - 1 : s_lo);
  const float s0 = A.scale0 * fm_norm_factor(A.fold0, bh, lane);
  const float gscale = QG ? fm_grad_scale(A.gpart ? A.gpart + int64_t(bh) * A.gnblk : nullptr, A.gnblk, lane) : 1.0f;
  const frag ones = M::splat(E(1.0f));
  fm_f32x16 acc[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) acc[s] = fm_zero16();
  for (int i = 0; i < cnt; ++i) {
    const int seg = suffix ? s_hi - 1 - i : s_lo + i;
    FM_SYNC();                                                         // the products of the segment before are done with the tiles
    if (QG) {
      r0.store(Lp, PQ, tid, s0);                                       // p = q'
      fm_o1_gh_rows<DH>(r1, ro, gi, gscale, Lr, PQ, Lc, nullptr, tid); // r = gh, weights c
    } else {
      r1.store(Lp, PQ, tid, 1.0f);                                     // p = v
      r0.store(Lr, PQ, tid, s0);                                       // r = k'
    }
    if (i + 1 < cnt) fetch(suffix ? seg - 1 : seg + 1);
    FM_SYNC();
    float* ds = sml + int64_t(seg) * O1Run<DH>::VS;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int t = wave + 4 * s;
      if (t >= NTILE) continue;
      // the sums of the run so far are this segment's state inside the run
      if (t < NT * NT) {
        float v[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) v[e] = acc[s][e];
        fm_put_small<E, DH>(A.b, big, nullptr, nullptr, seg, t, v, lr, lh);
      } else if (lr == 0) {
        const bool is_va = t < NT * NT + NT;
        float* dv = ds + (is_va ? 32 * (t - NT * NT) : DH + 32 * (t - NT * NT - NT));
        const float cf = is_va ? A.b.coefva : A.b.coefvb;
#pragma unroll
        for (int e = 0; e < 16; ++e) dv[fm_acc_row(e, lh)] = cf * acc[s][e];
      }
      // tiles of this wavefront: A operand (tile, feature offset), B operand (tile, or null = weights / ones)
      const E* ta = Lp; const E* tbt = nullptr;
      int fa = 0, fb = 0;
      bool wsum = false;
      if (t < NT * NT) { fa = 32 * (t / NT); tbt = Lr; fb = 32 * (t % NT); }
      else if (t < NT * NT + NT) { fa = 32 * (t - NT * NT); if (QG) wsum = true; else ta = Lr; }    // va: sum c q' | sum k'
      else { fa = 32 * (t - NT * NT - NT); if (QG) ta = Lr; }                                       // vb: sum gh   | sum v
#pragma unroll 4
      for (int k = 0; k < TT; k += M::KSTEP) {
        const frag a = M::load_tr(ta, PQ, k, fa, lane);
        const frag b = tbt ? M::load_tr(tbt, PQ, k, fb, lane) : (wsum ? M::load_perm(Lc + k, 0, lh) : ones);
        acc[s] = M::mma(a, b, acc[s]);
      }
    }
  }
  // the run's total, fp32
  float* tot = A.runtot + (int64_t(bh) * nruns + run) * O1Run<DH>::RS;
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int t = wave + 4 * s;
    if (t >= NTILE) continue;
    if (t < NT * NT) {
      const int rr = 32 * (t / NT), c = 32 * (t % NT) + lr;
#pragma unroll
      for (int e = 0; e < 16; ++e) tot[(rr + fm_acc_row(e, lh)) * DH + c] = A.b.coef1 * acc[s][e];
    } else if (lr == 0) {
      const bool is_va = t < NT * NT + NT;
      float* dv = tot + DH * DH + (is_va ? 32 * (t - NT * NT) : DH + 32 * (t - NT * NT - NT));
      const float cf = is_va ? A.b.coefva : A.b.coefvb;
#pragma unroll
      for (int e = 0; e < 16; ++e) dv[fm_acc_row(e, lh)] = cf * acc[s][e];
    }
  }
}

// Run totals -> for every run the sum over the runs before it (prefix) or after it (suffix), in place, and a
// compute-type copy of the slab part for the consumers' matrix operands.  grid (ceil(RS / 256), bh).
template <int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS) k_o1_runscan(float* FM_RESTRICT runtot, fm_half* FM_RESTRICT runhalf, int nruns, int suffix) {
  constexpr int RS = O1Run<DH>::RS, UB = 8;
  const int e = FM_BID_X * FM_THREADS + FM_TID_X, bh = FM_BID_Y;
  if (e >= RS) return;
  float* p = runtot + int64_t(bh) * nruns * RS + e;
  fm_half* h = runhalf + int64_t(bh) * nruns * DH * DH + e;
  float sum = 0.f;
  for (int b0 = 0; b0 < nruns; b0 += UB) {
    float t[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const int i = b0 + u, r = suffix ? nruns - 1 - i : i;
      t[u] = i < nruns ? p[int64_t(r) * RS] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const int i = b0 + u, r = suffix ? nruns - 1 - i : i;
      if (i < nruns) {
        p[int64_t(r) * RS] = sum;
        if (e < DH * DH) h[int64_t(r) * DH * DH] = CE<fm_half>::from(sum);
        sum += t[u];
      }
    }
  }
}
template <int DH> inline size_t fm_o1_sums_lds() { return (size_t(2) * FM_O1_SEG * (DH + Mma<fm_half>::PAD) + FM_O1_SEG) * 2; }

// ------------------------------------------------------------------------------
// k_o1_fwd: o and g of one segment.  grid (nseg, bh); wavefront w owns the 32 queries of tile w.
// The sums over the keys before the segment are two parts (see k_o1_sums): big / small, slot s: the segments before s
// inside its run; runbig / runtot, entry s / run_len: the runs before.  Slab [r][c] = a1 sum v_r k'_c, va = a1 sum k',
// vb = a0 sum v.
// ------------------------------------------------------------------------------
template <typename TIO> struct O1FwdArgs {
  TRef<const TIO> q, k, v;
  TRef<TIO> o; TRef<float> g;
  int n, nseg, nslots;
  const fm_half* big; const float* small;
  const fm_half* runbig; const float* runtot; int nruns, run_len;
  float a0, a1, sc;
  NormFold q_fold, k_fold;
};

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, 3) k_o1_fwd(O1FwdArgs<TIO> A) {
  typedef fm_half E;
  typedef TokCfg<E, DH, 1> C;
  typedef Mma<E> M;
  typedef TileMath<E> TM;
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, QW = C::QW, PQ = C::PQ, PS = C::PS;
  static_assert(QW == FM_O1_SEG, "one workgroup per segment");
  FM_DYN_SMEM(smem);
  E* Ks = reinterpret_cast<E*>(smem);                   // [QW][PQ] each; Q' lies in the first tile until its fragments are taken
  E* Vs = Ks + QW * PQ;
  float* vecs = reinterpret_cast<float*>(Vs + QW * PQ);  // va, vb of the prefix sums
  E* Sl = reinterpret_cast<E*>(vecs + 2 * DH);           // the prefix slab [DH][PS]
  E* Qs = Ks;
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  int seg, bh;
  fm_xcd_map(A.nseg, FM_GDIM_Y, seg, bh);
  const int t0 = seg * QW;
  const int own = wave * 32 + lr;
  // every load first: the three row tiles, the vector sums, the two parts of the prefix slab (16-byte chunks)
  constexpr int SCH = DH * DH / 8, SN = (SCH + FM_THREADS - 1) / FM_THREADS;
  O1Raw<DH> rk, rv;
  {
    O1Raw<DH> rq;
    frag rs[SN], rs2[SN];
    rq.load(A.q, bh, t0, A.n, tid); rk.load(A.k, bh, t0, A.n, tid); rv.load(A.v, bh, t0, A.n, tid);
    const int run = seg / A.run_len;
    float vsum = 0.f;
    if (tid < 2 * DH && seg > 0)
      vsum = A.small[(int64_t(bh) * A.nslots + seg) * O1Run<DH>::VS + tid] +
             A.runtot[(int64_t(bh) * A.nruns + run) * O1Run<DH>::RS + DH * DH + tid];
    const E* sl = A.big + (int64_t(bh) * A.nslots + seg) * StateDims<DH>::SLAB;
    const E* rl = A.runbig + (int64_t(bh) * A.nruns + run) * StateDims<DH>::SLAB;
#pragma unroll
    for (int i = 0; i < SN; ++i) {
      const int c = tid + FM_THREADS * i;
      if (SCH % FM_THREADS == 0 || c < SCH) {
        rs[i] = *reinterpret_cast<const frag*>(sl + c * 8);
        rs2[i] = *reinterpret_cast<const frag*>(rl + c * 8);
      }
    }
    if (tid < 2 * DH) vecs[tid] = vsum;
    rq.store(Qs, PQ, tid, A.sc * fm_norm_factor(A.q_fold, bh, lane));
#pragma unroll
    for (int i = 0; i < SN; ++i) {
      const int c = tid + FM_THREADS * i, row = c / (DH / 8), col = (c % (DH / 8)) * 8;
      if (SCH % FM_THREADS == 0 || c < SCH) *reinterpret_cast<frag*>(Sl + row * PS + col) = rs[i] + rs2[i];
    }
  }
  FM_SYNC();
  frag qf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) qf[ks] = M::load(Qs + own * PQ + ks * M::KSTEP + lh * M::KPL);
  FM_SYNC();                                             // every wavefront has its fragments of Q': K' takes the tile
  rk.store(Ks, PQ, tid, A.sc * fm_norm_factor(A.k_fold, bh, lane));
  rv.store(Vs, PQ, tid, 1.0f);
  FM_SYNC();
  fm_f32x16 acc[NT];
#pragma unroll
  for (int ct = 0; ct < NT; ++ct) acc[ct] = fm_zero16();
  float gsum = 0.f;
  if (seg > 0) {
    // the keys of the earlier segments: F += slab q', g += q' . va (this lane's half of the row; the halves meet below)
#pragma unroll
    for (int ct = 0; ct < NT; ++ct)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
        acc[ct] = M::mma(M::load(Sl + (32 * ct + lr) * PS + ks * M::KSTEP + lh * M::KPL), qf[ks], acc[ct]);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
      for (int i = 0; i < M::KPL; ++i) gsum += vecs[ks * M::KSTEP + lh * M::KPL + i] * M::elem(qf[ks], i);
  }
  const typename TM::Coef coef = TM::coef(A.a0, A.a1, 0.0f);
  for (int jt = 0; jt <= wave; ++jt) {
    fm_f32x16 s = fm_zero16();
    const E* krow = Ks + (32 * jt + lr) * PQ + lh * M::KPL;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) s = M::mma(M::load(krow + ks * M::KSTEP), qf[ks], s);
    frag pb[M::ACC_KSTEPS];
    // keys past the end of the sequence are zero rows, which the weight a0 would still count: the window ends at n - 1
    const int last = A.n - 1 - t0 - 32 * jt;
    const int hi = jt == wave ? (lr < last ? lr : last) : last;
    gsum += TM::fwd(s, coef, jt == wave || last < 31, 0, hi, lh, pb);
#pragma unroll
    for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
      for (int ct = 0; ct < NT; ++ct) acc[ct] = M::mma(M::load_tr(Vs, PQ, 32 * jt + 16 * ss, 32 * ct, lane), pb[ss], acc[ct]);
  }
  FM_SYNC();                                             // the tiles are spent: the output staging lies over them
  float* Os = reinterpret_cast<float*>(smem);           // [QW][fm_store_pitch]
  float gt = gsum + fm_shfl_xor(gsum, 32) + A.a0 * float(t0);
  const float ginv = 1.0f / gt;
  constexpr int OP = fm_store_pitch(DH);
#pragma unroll
  for (int ct = 0; ct < NT; ++ct)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int c = 32 * ct + fm_acc_row(4 * g, lh);
      fm_f32x4 w;
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = (acc[ct][4 * g + i] + vecs[DH + c + i]) * ginv;
      *reinterpret_cast<fm_f32x4*>(Os + own * OP + c) = w;
    }
  if (lh == 0 && t0 + own < A.n) A.g.base(bh)[int64_t(t0 + own) * A.g.s_n] = gt;
  FM_SYNC();
  TIO* ob = A.o.base(bh);
  for (int c = tid; c < QW * (DH / 8); c += FM_THREADS) {
    const int row = c / (DH / 8), col = (c % (DH / 8)) * 8;
    if (t0 + row < A.n) {
      const fm_f32x4 lo = *reinterpret_cast<const fm_f32x4*>(Os + row * OP + col);
      const fm_f32x4 hi = *reinterpret_cast<const fm_f32x4*>(Os + row * OP + col + 4);
      const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      IO<TIO>::st8(ob + int64_t(t0 + row) * A.o.s_n + col, A.o.vec != 0, v);
    }
  }
}
template <int DH> inline size_t fm_o1_fwd_lds() {
  // two row tiles, the two vectors and the prefix slab behind them; the output staging lies over the tiles
  const size_t tiles = size_t(2) * FM_O1_SEG * (DH + Mma<fm_half>::PAD) * 2 + size_t(2) * DH * 4 +
                       size_t(DH) * (DH + Mma<fm_half>::PAD) * 2;
  return tiles;
}

// ------------------------------------------------------------------------------
// k_o1_bwd: dq, dk and dv of one segment.  grid (nseg, bh); wavefront w owns the 32 tokens of tile w for all
// three.  First the tiles K', V, GH are in LDS (the raw q rows wait in registers): the prefix product and the
// dense tiles of dq, which is stored at once (its stores travel during the second phase); then Q' takes the place
// of K' for the dense tiles of dk and dv and the suffix products.
//   bigq (prefix, slot s: segments < s): slab [c][f] = a1 sum v_c k'_f, the forward's own state; smallq: va = a1 sum k'
//   bigk (suffix, slot s: segments > s): slab [f][c] = a1 sum q'_f gh_c;  smallk: va = a1 sum c q', vb = a0 sum gh
// each in two parts, the segments inside the run (big*, small*) and the whole runs (run*, see k_o1_sums), added on load.
// dq contracts the prefix slab over its first index and dv the suffix slab over its first index: a slab is staged
// in LDS with its rows in `tperm` order and those fragments are transposing reads, so no transposed copy of any
// state is ever written.
// ------------------------------------------------------------------------------
template <typename TIO> struct O1BwdArgs {
  TRef<const TIO> q, k, v, o, d_o; TRef<const float> g;
  TRef<TIO> dq, dk, dv;
  int n, nseg, nslots;
  const fm_half* bigq; const float* smallq;
  const fm_half* bigk; const float* smallk;
  const fm_half* runbigq; const float* runtotq;         // sums over whole runs: before the segment's run (q side) ...
  const fm_half* runbigk; const float* runtotk;         // ... and after it (k side)
  int nruns, run_len;
  float a0, a1, sc;
  const float* gpart; int gnblk;                        // see k_grad_scale
  NormFold q_fold, k_fold;                              // folded normalisation; bq / bk != null: its Jacobian (see TokArgs)
  float* bq; float* bk;
};

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, 2) k_o1_bwd(O1BwdArgs<TIO> A) {
  typedef fm_half E;
  typedef TokCfg<E, DH, 1> C;
  typedef Mma<E> M;
  typedef TileMath<E> TM;
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, QW = C::QW, PQ = C::PQ;
  FM_DYN_SMEM(smem);
  E* Ks = reinterpret_cast<E*>(smem);                   // [QW][PQ] each; Q' later lies over K'
  E* Vs = Ks + QW * PQ;
  E* Gs = Vs + QW * PQ;
  float* cs = reinterpret_cast<float*>(Gs + QW * PQ);    // [QW] c, fp32
  float* vecs = cs + QW;                                 // va of the prefix sums | va, vb of the suffix sums: 3 * DH
  E* Sl = reinterpret_cast<E*>(vecs + 3 * DH);           // one state slab [DH][PS], rows in `tperm` order
  E* Qs = Ks;
  constexpr int PS = C::PS;
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  int seg, bh;
  fm_xcd_map(A.nseg, FM_GDIM_Y, seg, bh);
  const int t0 = seg * QW;
  // a state slab (DH x DH, contiguous) as 16-byte chunks, DH / 32 per thread; into LDS with row r at tperm(r)
  constexpr int SCH = DH * DH / 8, SN = (SCH + FM_THREADS - 1) / FM_THREADS;
  auto slab_load = [&](const E* src, frag* r) {
#pragma unroll
    for (int i = 0; i < SN; ++i) {
      const int c = tid + FM_THREADS * i;
      if (SCH % FM_THREADS == 0 || c < SCH) r[i] = *reinterpret_cast<const frag*>(src + c * 8);
    }
  };
  // the two parts of a state, added
  auto slab_store = [&](const frag* r, const frag* r2) {
#pragma unroll
    for (int i = 0; i < SN; ++i) {
      const int c = tid + FM_THREADS * i, row = c / (DH / 8), col = (c % (DH / 8)) * 8;
      if (SCH % FM_THREADS == 0 || c < SCH) *reinterpret_cast<frag*>(Sl + M::tperm(row) * PS + col) = r[i] + r2[i];
    }
  };
  // Every load of the workgroup is issued before the first result is used: the five row tiles, the vector sums, the
  // fragments of the prefix state (this lane's rows of it), then the parts of the gradient scale and of the folds.
  O1Raw<DH> rq;
  frag rs[SN], rs2[SN];
  float gsc, qsc, ksc;
  const int run = seg / A.run_len;
  {
    O1Raw<DH> rk, rv, rdo, ro;
    rk.load(A.k, bh, t0, A.n, tid); rv.load(A.v, bh, t0, A.n, tid);
    rdo.load(A.d_o, bh, t0, A.n, tid); ro.load(A.o, bh, t0, A.n, tid);
    rq.load(A.q, bh, t0, A.n, tid);
    float gi[O1Raw<DH>::N];
#pragma unroll
    for (int i = 0; i < O1Raw<DH>::N; ++i) {
      const int row = t0 + O1Raw<DH>::row_of(i, tid);
      gi[i] = row < A.n ? A.g.base(bh)[int64_t(row) * A.g.s_n] : 1.0f;
    }
    float vsum = 0.f;
    if (tid < 3 * DH) {
      // the vector sums of the two states this segment reads (a segment at either end reads zeros instead)
      const bool pre = tid < DH;
      const int f = pre ? tid : tid - DH;
      const float* src = (pre ? A.smallq : A.smallk) + (int64_t(bh) * A.nslots + seg) * O1Run<DH>::VS + f;
      const float* src2 = (pre ? A.runtotq : A.runtotk) + (int64_t(bh) * A.nruns + run) * O1Run<DH>::RS + DH * DH + f;
      if (pre ? seg > 0 : seg < A.nseg - 1) vsum = *src + *src2;
    }
    slab_load(A.bigq + (int64_t(bh) * A.nslots + seg) * StateDims<DH>::SLAB, rs);
    slab_load(A.runbigq + (int64_t(bh) * A.nruns + run) * StateDims<DH>::SLAB, rs2);
    gsc = fm_grad_scale(A.gpart ? A.gpart + int64_t(bh) * A.gnblk : nullptr, A.gnblk, lane);
    qsc = A.sc * fm_norm_factor(A.q_fold, bh, lane);
    ksc = A.sc * fm_norm_factor(A.k_fold, bh, lane);
    if (tid < 3 * DH) vecs[tid] = vsum;
    slab_store(rs, rs2);
    rk.store(Ks, PQ, tid, ksc);
    rv.store(Vs, PQ, tid, 1.0f);
    fm_o1_gh_rows<DH>(rdo, ro, gi, gsc, Gs, PQ, nullptr, cs, tid);
  }
  FM_SYNC();

  const int own = wave * 32 + lr;                        // the lane's token inside the segment
  frag gf[NKS], kf[NKS], vf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    const int off = own * PQ + ks * M::KSTEP + lh * M::KPL;
    gf[ks] = M::load(Gs + off); kf[ks] = M::load(Ks + off); vf[ks] = M::load(Vs + off);
  }
  const float ci = cs[wave * 32 + lr];
  const typename TM::Coef coef = TM::coef(A.a0, A.a1, 0.0f);
  fm_f32x16 dq[NT], dk[NT], dv[NT];
#pragma unroll
  for (int mt = 0; mt < NT; ++mt) { dq[mt] = fm_zero16(); dk[mt] = fm_zero16(); dv[mt] = fm_zero16(); }
  const fm_f32x16 zero = fm_zero16();

  // the suffix slab travels to registers meanwhile; it takes the prefix slab's place after the first phase
  slab_load(A.bigk + (int64_t(bh) * A.nslots + seg) * StateDims<DH>::SLAB, rs);
  slab_load(A.runbigk + (int64_t(bh) * A.nruns + run) * StateDims<DH>::SLAB, rs2);
  // ---- dq: the keys of the earlier segments: sum_c slab[c][f] gh_c, transposing reads of the staged slab ----
  if (seg > 0) {
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) {
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) dq[mt] = M::mma(M::load_tr(Sl, PS, 16 * ks, 32 * mt, lane), gf[ks], dq[mt]);
#pragma unroll
      for (int e = 0; e < 16; ++e) dq[mt][e] -= ci * vecs[32 * mt + fm_acc_row(e, lh)];
    }
  }
  // ---- dq: dense tiles, own tokens as queries against the keys at or before them ----
  for (int jt = 0; jt <= wave; ++jt) {
    fm_f32x16 dp = fm_zero16();
    const E* vrow = Vs + (32 * jt + lr) * PQ + lh * M::KPL;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) dp = M::mma(M::load(vrow + ks * M::KSTEP), gf[ks], dp);
    frag db[M::ACC_KSTEPS];
    TM::dsc(zero, dp, -ci, coef, jt == wave, 0, lr, lh, db);         // diagonal tile: key row <= the lane's query
#pragma unroll
    for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) dq[mt] = M::mma(M::load_tr(Ks, PQ, 32 * jt + 16 * ss, 32 * mt, lane), db[ss], dq[mt]);
  }
  // A gradient leaves through an LDS region of the wavefront's own (its 32 tokens, 32 features at a time, already in
  // the output type): no barrier, so dq goes out right after its phase (its stores travel while dk and dv are
  // computed) and a wavefront that is done with dk and dv (the later its tokens, the fewer dense tiles) stores them
  // without waiting for the others.  (With the Jacobian of a folded normalisation, or rows that are not 16-byte
  // aligned, a gradient goes through the workgroup's fp32 staging at the end.)
  const float ginv = 1.0f / gsc;
  auto store_own = [&](const fm_f32x16* acc, float f, const TRef<TIO>& out) FM_ALWAYS_INLINE {
    if constexpr (sizeof(TIO) == 2) {
      constexpr int DP = FM_O1_DQ_PITCH;
      TIO* st = reinterpret_cast<TIO*>(Sl + DH * PS) + wave * 32 * DP;
      TIO* ob = out.base(bh);
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          fm_u32x2 w;
          w[0] = uint32_t(fm_f32_to_bf16(f * acc[mt][4 * g4])) | (uint32_t(fm_f32_to_bf16(f * acc[mt][4 * g4 + 1])) << 16);
          w[1] = uint32_t(fm_f32_to_bf16(f * acc[mt][4 * g4 + 2])) | (uint32_t(fm_f32_to_bf16(f * acc[mt][4 * g4 + 3])) << 16);
          *reinterpret_cast<fm_u32x2*>(st + lr * DP + fm_acc_row(4 * g4, lh)) = w;
        }
        FM_WAVE_SYNC();
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int c = lane + 64 * i, row = c >> 2, col = (c & 3) * 8;
          const int tok = t0 + wave * 32 + row;
          if (tok < A.n)
            *reinterpret_cast<fm_u32x4*>(ob + int64_t(tok) * out.s_n + 32 * mt + col) = *reinterpret_cast<const fm_u32x4*>(st + row * DP + col);
        }
        FM_WAVE_SYNC();
      }
    }
  };
  const bool dq_own = sizeof(TIO) == 2 && !A.bq && A.dq.vec != 0;
  const bool dk_own = sizeof(TIO) == 2 && !A.bk && A.dk.vec != 0;
  const bool dv_own = sizeof(TIO) == 2 && A.dv.vec != 0;
  if (dq_own) store_own(dq, A.sc * ginv, A.dq);
  FM_SYNC();                                             // K' and the prefix slab are spent
  rq.store(Qs, PQ, tid, qsc);
  slab_store(rs, rs2);
  FM_SYNC();
  // ---- dk, dv: dense tiles, own tokens as keys against the queries at or after them ----
  for (int it = wave; it < QW / 32; ++it) {
    fm_f32x16 s = fm_zero16(), dp = fm_zero16();
    const E* qrow = Qs + (32 * it + lr) * PQ + lh * M::KPL;
    const E* grow = Gs + (32 * it + lr) * PQ + lh * M::KPL;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      s = M::mma(M::load(qrow + ks * M::KSTEP), kf[ks], s);
      dp = M::mma(M::load(grow + ks * M::KSTEP), vf[ks], dp);
    }
    frag pb[M::ACC_KSTEPS], db[M::ACC_KSTEPS];
    float negc[16];                                      // -c of the tile's queries, the lane's 16 accumulator rows
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const fm_f32x4 t = *reinterpret_cast<const fm_f32x4*>(cs + 32 * it + 4 * lh + 8 * gq);
      negc[4 * gq] = -t[0]; negc[4 * gq + 1] = -t[1]; negc[4 * gq + 2] = -t[2]; negc[4 * gq + 3] = -t[3];
    }
    TM::both(s, dp, negc, coef, it == wave, lr, 31, lh, pb, db);     // diagonal tile: query row >= the lane's key
#pragma unroll
    for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) {
        dk[mt] = M::mma(M::load_tr(Qs, PQ, 32 * it + 16 * ss, 32 * mt, lane), db[ss], dk[mt]);
        dv[mt] = M::mma(M::load_tr(Gs, PQ, 32 * it + 16 * ss, 32 * mt, lane), pb[ss], dv[mt]);
      }
  }
  // ---- dk, dv: the queries of the later segments ----
  if (seg < A.nseg - 1) {
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) {
      // dk: sum_c slab[f][c] v_c (rows of the staged slab, at their permuted places); dv: sum_f slab[f][c] k'_f
      const E* srow = Sl + M::tperm(32 * mt + lr) * PS + lh * M::KPL;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        dk[mt] = M::mma(M::load(srow + ks * M::KSTEP), vf[ks], dk[mt]);
        dv[mt] = M::mma(M::load_tr(Sl, PS, 16 * ks, 32 * mt, lane), kf[ks], dv[mt]);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int f = 32 * mt + fm_acc_row(e, lh);
        dk[mt][e] -= vecs[DH + f];
        dv[mt][e] += vecs[2 * DH + f];
      }
    }
  }
  // ---- stores, through LDS.  With the Jacobian of a folded normalisation (bq / bk): the stored gradient carries
  // lim / max-norm and the workgroup's part of B = sum dy . y is left for k_norm_fix; the rows y * sc are the tiles
  // still in LDS (Q', and K' which is written back first) ----
  if (dk_own) store_own(dk, A.sc * ginv, A.dk);
  if (dv_own) store_own(dv, ginv, A.dv);
  if (dq_own && dk_own && dv_own) return;
  const int nblk = (A.n + QW - 1) / QW;
  const int xrow[1] = {own};
  float* Os = reinterpret_cast<float*>(Vs);              // over V and GH: [QW][fm_store_pitch] floats
  FM_SYNC();                                             // GH, V and c are spent
  if (!dq_own) {
    const float fac = A.bq ? fm_norm_factor(A.q_fold, bh, lane) : 1.0f;
    fm_store_tokens<TIO, E, DH, 1>(&dq, xrow, nullptr, A.sc * ginv * fac, Os, A.dq, bh, t0, A.n, tid,
                                   A.bq ? Qs : nullptr, fac > 0.f ? 1.0f / (fac * A.sc) : 0.f,
                                   A.bq ? A.bq + int64_t(bh) * nblk + seg : nullptr, PQ, t0);
  }
  if (A.bk) {
    // K' rows back into the tile (from the fragments every lane kept): the Jacobian part of dk needs them
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) *reinterpret_cast<frag*>(Ks + own * PQ + ks * M::KSTEP + lh * M::KPL) = kf[ks];
    FM_SYNC();
  }
  if (!dk_own) {
    const float fac = A.bk ? fm_norm_factor(A.k_fold, bh, lane) : 1.0f;
    fm_store_tokens<TIO, E, DH, 1>(&dk, xrow, nullptr, A.sc * ginv * fac, Os, A.dk, bh, t0, A.n, tid,
                                   A.bk ? Ks : nullptr, fac > 0.f ? 1.0f / (fac * A.sc) : 0.f,
                                   A.bk ? A.bk + int64_t(bh) * nblk + seg : nullptr, PQ, t0);
  }
  if (!dv_own) fm_store_tokens<TIO, E, DH, 1>(&dv, xrow, nullptr, ginv, Os, A.dv, bh, t0, A.n, tid);
}
template <int DH> inline size_t fm_o1_bwd_lds() {
  const size_t tile = size_t(FM_O1_SEG) * (DH + Mma<fm_half>::PAD) * 2;
  const size_t tiles = 3 * tile + size_t(FM_O1_SEG) * 4 + size_t(3) * DH * 4 + size_t(DH) * (DH + Mma<fm_half>::PAD) * 2 +
                       size_t(FM_THREADS / 64) * 32 * FM_O1_DQ_PITCH * 2;            // and the wavefronts' own output staging
  const size_t outst = tile + size_t(FM_O1_SEG) * fm_store_pitch(DH) * 4;      // Q' / K' tile kept, staging over V and GH
  return tiles > outst ? tiles : outst;
}
