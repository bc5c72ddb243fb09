// Order 1, long sequences: the three gradients of one 128-token segment in one pass.
//
// With f(s) = a0 + a1 s the score gradient does not depend on the score, dS_ij = a1 (gh_i.v_j - c_i), and every
// term that crosses a segment boundary is a D x D sum:
//     dq'_i = a1 [ (sum_{j<=i} k'_j v_j^T) gh_i - c_i sum_{j<=i} k'_j ]
//     dk'_j = a1 [ (sum_{i>=j} q'_i gh_i^T) v_j - sum_{i>=j} c_i q'_i ]
//     dv_j  = a0 sum_{i>=j} gh_i + a1 (sum_{i>=j} gh_i q'_i^T) k'_j
// so a segment needs its own 128 rows of q', k', v, gh (and c), the prefix sums of (k', v) before it and the
// suffix sums of (q', gh) after it, and nothing else.  One workgroup per segment stages the four row tiles in
// LDS once (74 KB: two workgroups per CU, so one loads while the other computes), each wavefront owns 32 tokens
// and accumulates dq, dk and dv for them: the dense causal tiles inside the segment (8 matrix instructions per
// tile pair for dq, 16 for dk and dv), then the three state products.  The kernel is bound by the bytes it
// moves: four tensors in, three out, 16 KB of states per segment; the separate dQ, dK and dV kernels read the
// four tensors three times over and stream every tile of a segment again per 128 own tokens.
// Replaces, for this case, calc_gradq/k/v_masked (fastmax_cuda_backward.cu:101-188, 272-358, 430-491).
#pragma once
#include "fm_tok.h"

template <typename TIO, typename E> struct O1BwdArgs {
  const E* qr; const E* gh; const E* kr; const E* vr;   // [bh][npad][DH] compute-type rows (q', gh, k', v)
  const E* cv;                                          // [bh][npad] c, 16-token groups in `tperm` order
  int npad, n, nseg, nslots;
  const E* bigq; const float* smallq;                   // prefix sums of (k', v): slab [f][c] = a1 sum k'_f v_c; va = a1 sum k'
  const E* bigk; const float* smallk;                   // suffix sums of (q', gh): slab [f][c] = a1 sum q'_f gh_c; va = a1 sum c q'; vb = a0 sum gh
  const E* bigv;                                        // the same slab transposed: [c][f]
  TRef<TIO> dq, dk, dv;
  float a0, a1, sc;
  const float* gpart; int gnblk;                        // see k_grad_scale
  NormFold q_fold, k_fold;                              // Jacobian of a folded normalisation: see TokArgs
  float* bq; float* bk;
};

template <typename TIO, typename E, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, 2) k_o1_bwd(O1BwdArgs<TIO, E> A) {
  typedef TokCfg<E, DH, 1> C;
  typedef Mma<E> M;
  typedef TileMath<E> TM;
  typedef typename M::frag frag;
  static_assert(M::HAS_TR, "this kernel reads transposed fragments out of row tiles");
  constexpr int NT = C::NT, NKS = C::NKS, QW = C::QW, PQ = C::PQ;   // QW = 128 tokens = one segment
  FM_DYN_SMEM(smem);
  E* Qs = reinterpret_cast<E*>(smem);                   // [QW][PQ] each
  E* Gs = Qs + QW * PQ;
  E* Ks = Gs + QW * PQ;
  E* Vs = Ks + QW * PQ;
  E* cs = Vs + QW * PQ;                                  // [QW] c in `tperm` order
  float* vecs = reinterpret_cast<float*>(cs + QW);       // va of the prefix sums | va, vb of the suffix sums: 3 * DH
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  int seg, bh;
  fm_xcd_map(A.nseg, FM_GDIM_Y, seg, bh);
  const int t0 = seg * QW;
  const int64_t rows = (int64_t(bh) * A.npad + t0) * DH;
  {
    TileRegs<E, QW, DH> rq, rg, rk, rv;
    rq.load(A.qr + rows, DH, tid); rg.load(A.gh + rows, DH, tid);
    rk.load(A.kr + rows, DH, tid); rv.load(A.vr + rows, DH, tid);
    if (tid < QW) cs[tid] = A.cv[int64_t(bh) * A.npad + t0 + tid];
    if (tid < 3 * DH) {
      // the vector sums of the two states this segment reads (a segment at either end reads zeros instead)
      const bool pre = tid < DH;
      const float* src = (pre ? A.smallq : A.smallk) + (int64_t(bh) * A.nslots + seg) * StateDims<DH>::SMALL + DH * DH +
                         (pre ? tid : tid - DH);
      vecs[tid] = (pre ? seg > 0 : seg < A.nseg - 1) ? *src : 0.f;
    }
    rq.store(Qs, PQ, tid); rg.store(Gs, PQ, tid); rk.store(Ks, PQ, tid); rv.store(Vs, PQ, tid);
  }
  const float gsc = fm_grad_scale(A.gpart ? A.gpart + int64_t(bh) * A.gnblk : nullptr, A.gnblk, lane);
  FM_SYNC();

  const int own = wave * 32 + lr;                        // the lane's token inside the segment
  frag qf[NKS], gf[NKS], kf[NKS], vf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    const int off = own * PQ + ks * M::KSTEP + lh * M::KPL;
    qf[ks] = M::load(Qs + off); gf[ks] = M::load(Gs + off); kf[ks] = M::load(Ks + off); vf[ks] = M::load(Vs + off);
  }
  const float ci = float(cs[wave * 32 + M::tperm(lr)]);
  const typename TM::CSplat csp = TM::splat_c(ci);
  const typename TM::Coef coef = TM::coef(A.a0, A.a1, 0.0f);
  fm_f32x16 dq[NT], dk[NT], dv[NT];
#pragma unroll
  for (int mt = 0; mt < NT; ++mt) { dq[mt] = fm_zero16(); dk[mt] = fm_zero16(); dv[mt] = fm_zero16(); }
  const fm_f32x16 zero = fm_zero16();

  // ---- the sums over the other segments first (their loads have the longest way): fragments straight from
  // the states, which the L2 holds ----
  const int frag_off = lr * DH + lh * M::KPL;
  if (seg > 0) {
    const E* sq = A.bigq + (int64_t(bh) * A.nslots + seg) * StateDims<DH>::SLAB + frag_off;
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) {
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) dq[mt] = M::mma(M::load(sq + 32 * mt * DH + ks * M::KSTEP), gf[ks], dq[mt]);
#pragma unroll
      for (int e = 0; e < 16; ++e) dq[mt][e] -= ci * vecs[32 * mt + fm_acc_row(e, lh)];
    }
  }
  if (seg < A.nseg - 1) {
    const E* sk = A.bigk + (int64_t(bh) * A.nslots + seg) * StateDims<DH>::SLAB + frag_off;
    const E* sv = A.bigv + (int64_t(bh) * A.nslots + seg) * StateDims<DH>::SLAB + frag_off;
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) {
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        dk[mt] = M::mma(M::load(sk + 32 * mt * DH + ks * M::KSTEP), vf[ks], dk[mt]);
        dv[mt] = M::mma(M::load(sv + 32 * mt * DH + ks * M::KSTEP), kf[ks], dv[mt]);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int f = 32 * mt + fm_acc_row(e, lh);
        dk[mt][e] -= vecs[DH + f];
        dv[mt][e] += vecs[2 * DH + f];
      }
    }
  }
  // ---- dense tiles: own tokens as queries against the keys at or before them ----
  for (int jt = 0; jt <= wave; ++jt) {
    fm_f32x16 dp = fm_zero16();
    const E* vrow = Vs + (32 * jt + lr) * PQ + lh * M::KPL;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) dp = M::mma(M::load(vrow + ks * M::KSTEP), gf[ks], dp);
    frag db[M::ACC_KSTEPS];
    TM::dsc(zero, dp, csp, coef, jt == wave, 0, lr, lh, db);         // diagonal tile: key row <= the lane's query
#pragma unroll
    for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) dq[mt] = M::mma(M::load_tr(Ks, PQ, 32 * jt + 16 * ss, 32 * mt, lane), db[ss], dq[mt]);
  }
  // ---- dense tiles: own tokens as keys against the queries at or after them ----
  for (int it = wave; it < QW / 32; ++it) {
    fm_f32x16 s = fm_zero16(), dp = fm_zero16();
    const E* qrow = Qs + (32 * it + lr) * PQ + lh * M::KPL;
    const E* grow = Gs + (32 * it + lr) * PQ + lh * M::KPL;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      s = M::mma(M::load(qrow + ks * M::KSTEP), kf[ks], s);
      dp = M::mma(M::load(grow + ks * M::KSTEP), vf[ks], dp);
    }
    frag crow[M::ACC_KSTEPS], pb[M::ACC_KSTEPS], db[M::ACC_KSTEPS];
#pragma unroll
    for (int ss = 0; ss < M::ACC_KSTEPS; ++ss) crow[ss] = M::load_perm(cs + 32 * it, ss, lh);
    TM::both(s, dp, crow, coef, it == wave, lr, 31, lh, pb, db);     // diagonal tile: query row >= the lane's key
#pragma unroll
    for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) {
        dk[mt] = M::mma(M::load_tr(Qs, PQ, 32 * it + 16 * ss, 32 * mt, lane), db[ss], dk[mt]);
        dv[mt] = M::mma(M::load_tr(Gs, PQ, 32 * it + 16 * ss, 32 * mt, lane), pb[ss], dv[mt]);
      }
  }
  FM_SYNC();                                             // the row tiles are spent: the output staging lies over them
  // ---- stores, through LDS; with a folded normalisation the Jacobian's pieces as in k_ds ----
  float* Os = reinterpret_cast<float*>(smem);
  const int xrow[1] = {own};
  const float ginv = 1.0f / gsc;
  const int nblk = (A.n + QW - 1) / QW;
  {
    const float fac = A.bq ? fm_norm_factor(A.q_fold, bh, lane) : 1.0f;
    fm_store_tokens<TIO, E, DH, 1>(&dq, xrow, nullptr, A.sc * ginv * fac, Os, A.dq, bh, t0, A.n, tid,
                                   A.bq ? A.qr + int64_t(bh) * A.npad * DH : nullptr, fac > 0.f ? 1.0f / (fac * A.sc) : 0.f,
                                   A.bq ? A.bq + int64_t(bh) * nblk + seg : nullptr);
  }
  {
    const float fac = A.bk ? fm_norm_factor(A.k_fold, bh, lane) : 1.0f;
    fm_store_tokens<TIO, E, DH, 1>(&dk, xrow, nullptr, A.sc * ginv * fac, Os, A.dk, bh, t0, A.n, tid,
                                   A.bk ? A.kr + int64_t(bh) * A.npad * DH : nullptr, fac > 0.f ? 1.0f / (fac * A.sc) : 0.f,
                                   A.bk ? A.bk + int64_t(bh) * nblk + seg : nullptr);
  }
  fm_store_tokens<TIO, E, DH, 1>(&dv, xrow, nullptr, ginv, Os, A.dv, bh, t0, A.n, tid);
}

template <typename E, int DH> inline size_t fm_o1_bwd_lds() {
  typedef TokCfg<E, DH, 1> C;
  const size_t tiles = (size_t(4) * C::QW * C::PQ + C::QW) * sizeof(E) + size_t(3) * DH * 4;
  const size_t outst = size_t(C::QW) * (DH + 1) * 4;
  return tiles > outst ? tiles : outst;
}
