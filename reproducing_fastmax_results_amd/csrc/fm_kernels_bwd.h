// Backward kernels.  With x_ij = q_i.k_j, f(x) = a0 + c1 x + c2 x^2 and, per query,
//     gh_i = dO_i / g_i,   c_i = gh_i . o_i,
//     dS_ij = M_ij (c1 + 2 c2 x_ij) (gh_i . v_j - c_i),
//     dQ_i = sum_j dS_ij k_j,   dK_j = sum_i dS_ij q_i,   dV_j = sum_i M_ij f(x_ij) gh_i
// (fastattention_einops.py:384-691; fastmax_cuda_backward.cu:26-491 computes the same
// sums with one thread per feature and serial loops over tokens).  Tokens of other
// segments contribute through moment states exactly as in the forward:
//   dQ: prefix states of (k, k, v)  contracted with (q, gh)
//   dK: suffix states of (q, q, gh) contracted with (k, v)
//   dV: suffix states of (q, gh, q) contracted with (k, k)
// and tokens of the same segment through dense masked tiles.
#pragma once
#include "fm_kernels.h"

template <typename TIO, typename E> struct BwdArgs {
  TRef<const TIO> q, k, v;
  TRef<TIO> dq, dk, dv;
  const E* gh; const E* ght; const E* qt; const E* qr; const E* kt; const E* kr; const E* vr; const E* cv;   // workspace copies
  int npad_q, npad_k;
  const E* bigq; const float* smallq;      // prefix (k, k, v)
  const E* bigk; const float* smallk;      // suffix (q, q, gh)
  const E* bigv; const float* smallv;      // suffix (q, gh, q)
  int nslots;
  int nq, nk, L, nseg, causal, use_state, quad;
  float a0, a1, a2;
  float sc;                                // sqrt(1/tau): q and k are used as sc*q, sc*k
  float gscale;                            // power of two folded into gh and c by k_prep_bwd
  float zscale_q;                          // factor on the Z of the (k, k, v) state (2 when the forward's state is reused)
};

// Z (fp32, [DH][DH]) -> LDS in the compute type (hi/lo split for _Float16), va/vb -> vecs.
template <typename E, int DH, int QT>
FM_DEVICE void fm_stage_small(const float* sml, E* Zs, float* vecs, int tid, float zscale = 1.0f) {
  typedef TokCfg<E, DH, QT> C;
  for (int i = tid; i < DH * DH; i += FM_THREADS) {
    const float z = sml[i] * zscale;
    const int r = i / DH, c = i % DH;
    const E hi = CE<E>::from(z);
    Zs[r * C::PS + c] = hi;
    if (C::NZ == 2) Zs[DH * C::PS + r * C::PS + c] = CE<E>::from(z - float(hi));
  }
  if (tid < 2 * DH) vecs[tid] = sml[DH * DH + tid];
}

// y[mt] (rows m, column = token) = sum_l Z[m][l] * tok_l, from the staged Z and the
// token's B fragments.
template <typename E, int DH, int QT>
FM_DEVICE fm_f32x16 fm_zy(const E* Zs, const typename Mma<E>::frag* tf, int mt, int lr, int lh) {
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  fm_f32x16 y = fm_zero16();
#pragma unroll
  for (int z = 0; z < C::NZ; ++z)
#pragma unroll
    for (int ks = 0; ks < C::NKS; ++ks)
      y = M::mma(M::load(Zs + z * DH * C::PS + (32 * mt + lr) * C::PS + ks * M::KSTEP + lh * M::KPL), tf[ks], y);
  return y;
}

// Accumulators (rows = feature, column = token of tile j) -> caller tensor rows, through LDS.
template <typename TIO, typename E, int DH, int QT>
FM_DEVICE void fm_store_tokens(fm_f32x16 (*acc)[DH / 32], const int* xrow, const float* addvec, float scale, float* Os,
                               TRef<TIO> out, int bh, int row0, int nrows, int tid) {
  typedef TokCfg<E, DH, QT> C;
  const int lane = tid & 63, lh = lane >> 5;
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int ct = 0; ct < C::NT; ++ct)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int c = 32 * ct + fm_acc_row(e, lh);
        Os[xrow[j] * (DH + 1) + c] = scale * (acc[j][ct][e] + (addvec ? addvec[c] : 0.f));
      }
  FM_SYNC();
  TIO* ob = out.p + int64_t(bh) * out.s_bh;
  for (int c = tid; c < C::QW * (DH / 8); c += FM_THREADS) {
    const int row = c / (DH / 8), col = (c % (DH / 8)) * 8;
    if (row0 + row < nrows) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = Os[row * (DH + 1) + col + i];
      IO<TIO>::st8(ob + int64_t(row0 + row) * out.s_n + col, out.vec != 0, v);
    }
  }
  FM_SYNC();
}

// ------------------------------------------------------------------------------
// k_dq: gradient with respect to one block of QW queries.  grid (ceil(nq/QW), bh).
// ------------------------------------------------------------------------------
template <typename TIO, typename E, int DH, int QT>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS) k_dq(BwdArgs<TIO, E> A) {
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  typedef TileMath<E> TM;
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, QW = C::QW, PQ = C::PQ, KT = C::KT, PV = C::PV;
  constexpr int NBUF = sizeof(E) == 2 ? 2 : 1;
  constexpr int STAGE = 2 * KT * PQ + DH * PV;        // K rows, V rows, K transposed
  FM_DYN_SMEM(smem);
  E* Qs = reinterpret_cast<E*>(smem);                 // [QW][PQ]  q rows
  E* Gs = Qs + QW * PQ;                               // [QW][PQ]  gh rows
  float* vecs = reinterpret_cast<float*>(Gs + QW * PQ);
  E* R = reinterpret_cast<E*>(vecs + 2 * DH);         // Z | slabs | dense tiles | output staging
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  const int nqb = FM_GDIM_X;
  int unit, bh;
  fm_xcd_map(nqb, FM_GDIM_Y, unit, bh);
  const int qb = A.causal ? (nqb - 1 - unit) : unit;
  const int q0 = qb * QW;
  const int seg = A.causal ? q0 / A.L : 0;
  const bool use_state = A.use_state && (!A.causal || seg > 0);
  const int slot = A.causal ? seg : 0;
  const int kbeg = A.causal ? seg * A.L : 0;
  const int kend = A.causal ? (q0 + QW < A.nk ? q0 + QW : A.nk) : (A.use_state ? 0 : A.nk);

  {
    RowRegs<TIO, E, QW, DH> rq;
    rq.load(A.q.p + int64_t(bh) * A.q.s_bh, A.q.s_n, A.q.vec != 0, q0, A.nq, tid);
    rq.store(Qs, PQ, tid, A.sc);
    TileRegs<E, QW, DH> rg;                            // gh rows are dense [npad_q][DH]
    rg.load(A.gh + (int64_t(bh) * A.npad_q + q0) * DH, DH, tid);
    rg.store(Gs, PQ, tid);
  }
  if (use_state)
    fm_stage_small<E, DH, QT>(A.smallq + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL, R, vecs, tid, A.zscale_q);
  FM_SYNC();

  int tw[QT], xrow[QT];
  float ci[QT];
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    tw[j] = (j == 0) ? wave : (4 * QT - 1 - wave);
    xrow[j] = tw[j] * 32 + lr;
    ci[j] = float(A.cv[int64_t(bh) * A.npad_q + q0 + M::tperm(xrow[j])]);   // c is stored in tile order
  }
  frag qf[QT][NKS], gf[QT][NKS];
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      qf[j][ks] = M::load(Qs + xrow[j] * PQ + ks * M::KSTEP + lh * M::KPL);
      gf[j][ks] = M::load(Gs + xrow[j] * PQ + ks * M::KSTEP + lh * M::KPL);
    }
  fm_f32x16 acc[QT][NT];
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) acc[j][mt] = fm_zero16();

  if (use_state) {
    // - c_i * (va[m] + sum_l Z[m][l] q_il)
#pragma unroll
    for (int j = 0; j < QT; ++j)
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) {
        const fm_f32x16 y = fm_zy<E, DH, QT>(R, qf[j], mt, lr, lh);
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][mt][e] = -ci[j] * (y[e] + vecs[32 * mt + fm_acc_row(e, lh)]);
      }
    FM_SYNC();                                         // Z is overwritten by the slabs
    const E* state = A.bigq + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::BIG;
    fm_readout<E, DH, QT, NT>(state, A.quad != 0, Qs, xrow, gf, R, acc, tid);
  }

  if (kend > kbeg) {
    const typename TM::Coef coef = TM::coef(A.a0, A.a1, A.a2);
    TileRegs<E, KT, DH> rk, rv;
    TileRegs<E, DH, KT> rkt;
    const E* kb = A.kr + int64_t(bh) * A.npad_k * DH;
    const E* vb = A.vr + int64_t(bh) * A.npad_k * DH;
    const E* ktb = A.kt + int64_t(bh) * DH * A.npad_k;
    rk.load(kb + int64_t(kbeg) * DH, DH, tid);
    rv.load(vb + int64_t(kbeg) * DH, DH, tid);
    rkt.load(ktb + kbeg, A.npad_k, tid);
    int buf = 0;
    for (int kt0 = kbeg; kt0 < kend; kt0 += KT) {
      E* Ks = R + buf * STAGE; E* Vs = Ks + KT * PQ; E* Kts = Vs + KT * PQ;
      rk.store(Ks, PQ, tid); rv.store(Vs, PQ, tid); rkt.store(Kts, PV, tid);
      FM_SYNC();
      if (kt0 + KT < kend) {
        rk.load(kb + int64_t(kt0 + KT) * DH, DH, tid);
        rv.load(vb + int64_t(kt0 + KT) * DH, DH, tid);
        rkt.load(ktb + kt0 + KT, A.npad_k, tid);
      }
      constexpr int NI = (KT / 32) * QT;
      bool act[NI];
#pragma unroll
      for (int it = 0; it < NI; ++it) {
        const int key0 = kt0 + 32 * (it / QT), qlo = q0 + tw[it % QT] * 32;
        act[it] = key0 < kend && !(A.causal && key0 > qlo + 31);
      }
      fm_f32x16 s_cur, dp_cur;
      if (act[0]) {
        s_cur = fm_zero16(); dp_cur = fm_zero16();
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          s_cur = M::mma(M::load(Ks + lr * PQ + ks * M::KSTEP + lh * M::KPL), qf[0][ks], s_cur);
          dp_cur = M::mma(M::load(Vs + lr * PQ + ks * M::KSTEP + lh * M::KPL), gf[0][ks], dp_cur);
        }
      }
#pragma unroll
      for (int it = 0; it < NI; ++it) {
        const int st = it / QT, j = it % QT;
        fm_f32x16 s_nxt, dp_nxt;
        if (it + 1 < NI && act[(it + 1 < NI) ? it + 1 : it]) {
          s_nxt = fm_zero16(); dp_nxt = fm_zero16();
          const int st2 = (it + 1) / QT, j2 = (it + 1) % QT;
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            s_nxt = M::mma(M::load(Ks + (32 * st2 + lr) * PQ + ks * M::KSTEP + lh * M::KPL), qf[j2][ks], s_nxt);
            dp_nxt = M::mma(M::load(Vs + (32 * st2 + lr) * PQ + ks * M::KSTEP + lh * M::KPL), gf[j2][ks], dp_nxt);
          }
        }
        if (act[it]) {
          const int key0 = kt0 + 32 * st, qlo = q0 + tw[j] * 32;
          const bool edge = (A.causal && key0 + 31 > qlo) || (key0 + 31 >= A.nk);
          int hi = A.nk - 1 - key0;
          if (A.causal && qlo + lr - key0 < hi) hi = qlo + lr - key0;
          frag db[M::ACC_KSTEPS];
          frag kf[NT][M::ACC_KSTEPS];
#pragma unroll
          for (int mt = 0; mt < NT; ++mt)
#pragma unroll
            for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
              kf[mt][ss] = M::load_perm(Kts + (32 * mt + lr) * PV + 32 * st, ss, lh);
          TM::dsc(s_cur, dp_cur, TM::splat_c(ci[j]), coef, edge, 0, hi, lh, db);
#pragma unroll
          for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
            for (int mt = 0; mt < NT; ++mt) acc[j][mt] = M::mma(kf[mt][ss], db[ss], acc[j][mt]);
        }
        s_cur = s_nxt; dp_cur = dp_nxt;
      }
      if (NBUF == 1) FM_SYNC(); else buf ^= 1;
    }
    if (NBUF == 2) FM_SYNC();
  }
  fm_store_tokens<TIO, E, DH, QT>(acc, xrow, nullptr, A.sc / A.gscale, reinterpret_cast<float*>(R), A.dq, bh, q0, A.nq, tid);
}

// ------------------------------------------------------------------------------
// k_dkv: gradients with respect to one block of QW keys/values.  grid (ceil(nk/QW), bh).
// ------------------------------------------------------------------------------
template <typename TIO, typename E, int DH, int QT>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS) k_dkv(BwdArgs<TIO, E> A) {
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  typedef TileMath<E> TM;
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, KW = C::QW, PQ = C::PQ, KT = C::KT, PV = C::PV;
  constexpr int NBUF = sizeof(E) == 2 ? 2 : 1;
  constexpr int STAGE = 2 * KT * PQ + 2 * DH * PV;     // q rows, gh rows, q transposed, gh transposed
  constexpr int STAGE_PAD = STAGE + 2 * KT;            // + c values (compute type, padded)
  FM_DYN_SMEM(smem);
  E* Ks = reinterpret_cast<E*>(smem);                 // [KW][PQ]  k rows
  E* Vs = Ks + KW * PQ;                               // [KW][PQ]  v rows
  float* vecs = reinterpret_cast<float*>(Vs + KW * PQ);   // va, vb of the (q, q, gh) state
  E* R = reinterpret_cast<E*>(vecs + 2 * DH);
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  int unit, bh;
  fm_xcd_map(FM_GDIM_X, FM_GDIM_Y, unit, bh);
  const int k0 = unit * KW;                            // early key blocks are the heavy ones
  const int seg = A.causal ? k0 / A.L : 0;
  const bool use_state = A.use_state && (!A.causal || seg < A.nseg - 1);
  const int slot = A.causal ? seg : 0;
  const int ibeg = A.causal ? k0 : 0;
  const int iend = A.causal ? ((seg + 1) * A.L < A.nq ? (seg + 1) * A.L : A.nq) : (A.use_state ? 0 : A.nq);

  {
    RowRegs<TIO, E, KW, DH> rk;
    rk.load(A.k.p + int64_t(bh) * A.k.s_bh, A.k.s_n, A.k.vec != 0, k0, A.nk, tid);
    rk.store(Ks, PQ, tid, A.sc);
    rk.load(A.v.p + int64_t(bh) * A.v.s_bh, A.v.s_n, A.v.vec != 0, k0, A.nk, tid);
    rk.store(Vs, PQ, tid, 1.0f);
  }
  if (use_state)
    fm_stage_small<E, DH, QT>(A.smallk + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL, R, vecs, tid);
  FM_SYNC();

  int tw[QT], xrow[QT];
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    tw[j] = (j == 0) ? wave : (4 * QT - 1 - wave);
    xrow[j] = tw[j] * 32 + lr;
  }
  frag kf[QT][NKS], vf[QT][NKS];
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      kf[j][ks] = M::load(Ks + xrow[j] * PQ + ks * M::KSTEP + lh * M::KPL);
      vf[j][ks] = M::load(Vs + xrow[j] * PQ + ks * M::KSTEP + lh * M::KPL);
    }
  fm_f32x16 ak[QT][NT], av[QT][NT];
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) { ak[j][mt] = fm_zero16(); av[j][mt] = fm_zero16(); }

  if (use_state) {
    // dK: - (va[m] + sum_l Zc[m][l] k_jl)
#pragma unroll
    for (int j = 0; j < QT; ++j)
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) {
        const fm_f32x16 y = fm_zy<E, DH, QT>(R, kf[j], mt, lr, lh);
#pragma unroll
        for (int e = 0; e < 16; ++e) ak[j][mt][e] = -(y[e] + vecs[32 * mt + fm_acc_row(e, lh)]);
      }
    FM_SYNC();
    const int64_t so = (int64_t(bh) * A.nslots + slot) * StateDims<DH>::BIG;
    fm_readout<E, DH, QT, NT>(A.bigk + so, A.quad != 0, Ks, xrow, vf, R, ak, tid);
    fm_readout<E, DH, QT, NT>(A.bigv + so, A.quad != 0, Ks, xrow, kf, R, av, tid);
  }

  if (iend > ibeg) {
    const typename TM::Coef coef = TM::coef(A.a0, A.a1, A.a2);
    TileRegs<E, KT, DH> rq, rg;
    TileRegs<E, DH, KT> rqt, rgt;
    const E* qb = A.qr + int64_t(bh) * A.npad_q * DH;
    const E* ghb = A.gh + int64_t(bh) * A.npad_q * DH;
    const E* qtb = A.qt + int64_t(bh) * DH * A.npad_q;
    const E* gtb = A.ght + int64_t(bh) * DH * A.npad_q;
    const E* cvb = A.cv + int64_t(bh) * A.npad_q;
    E creg = E(0.f);
    rq.load(qb + int64_t(ibeg) * DH, DH, tid);
    rg.load(ghb + int64_t(ibeg) * DH, DH, tid);
    rqt.load(qtb + ibeg, A.npad_q, tid);
    rgt.load(gtb + ibeg, A.npad_q, tid);
    if (tid < KT) creg = cvb[ibeg + tid];
    int buf = 0;
    for (int i0 = ibeg; i0 < iend; i0 += KT) {
      E* Qr = R + buf * STAGE_PAD; E* Gr = Qr + KT * PQ; E* Qts = Gr + KT * PQ; E* Gts = Qts + DH * PV;
      E* cs = Gts + DH * PV;
      rq.store(Qr, PQ, tid); rg.store(Gr, PQ, tid); rqt.store(Qts, PV, tid); rgt.store(Gts, PV, tid);
      if (tid < KT) cs[tid] = creg;
      FM_SYNC();
      if (i0 + KT < iend) {
        rq.load(qb + int64_t(i0 + KT) * DH, DH, tid);
        rg.load(ghb + int64_t(i0 + KT) * DH, DH, tid);
        rqt.load(qtb + i0 + KT, A.npad_q, tid);
        rgt.load(gtb + i0 + KT, A.npad_q, tid);
        if (tid < KT) creg = cvb[i0 + KT + tid];
      }
      constexpr int NI = (KT / 32) * QT;
      bool act[NI];
#pragma unroll
      for (int it = 0; it < NI; ++it) {
        const int qi0 = i0 + 32 * (it / QT), klo = k0 + tw[it % QT] * 32;
        act[it] = qi0 < iend && !(A.causal && qi0 + 31 < klo);   // skip queries that precede all keys
      }
      fm_f32x16 s_cur, dp_cur;
      if (act[0]) {
        s_cur = fm_zero16(); dp_cur = fm_zero16();
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          s_cur = M::mma(M::load(Qr + lr * PQ + ks * M::KSTEP + lh * M::KPL), kf[0][ks], s_cur);
          dp_cur = M::mma(M::load(Gr + lr * PQ + ks * M::KSTEP + lh * M::KPL), vf[0][ks], dp_cur);
        }
      }
#pragma unroll
      for (int it = 0; it < NI; ++it) {
        const int st = it / QT, j = it % QT;
        fm_f32x16 s_nxt, dp_nxt;
        if (it + 1 < NI && act[(it + 1 < NI) ? it + 1 : it]) {
          s_nxt = fm_zero16(); dp_nxt = fm_zero16();
          const int st2 = (it + 1) / QT, j2 = (it + 1) % QT;
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            s_nxt = M::mma(M::load(Qr + (32 * st2 + lr) * PQ + ks * M::KSTEP + lh * M::KPL), kf[j2][ks], s_nxt);
            dp_nxt = M::mma(M::load(Gr + (32 * st2 + lr) * PQ + ks * M::KSTEP + lh * M::KPL), vf[j2][ks], dp_nxt);
          }
        }
        if (act[it]) {
          const int qi0 = i0 + 32 * st, klo = k0 + tw[j] * 32;
          const bool edge = (A.causal && qi0 < klo + 31) || (qi0 + 31 >= A.nq);
          const int lo = A.causal ? klo + lr - qi0 : 0;
          const int hi = A.nq - 1 - qi0;
          frag pb[M::ACC_KSTEPS], db[M::ACC_KSTEPS], crow[M::ACC_KSTEPS];
          frag gtf[NT][M::ACC_KSTEPS], qtf[NT][M::ACC_KSTEPS];
#pragma unroll
          for (int ss = 0; ss < M::ACC_KSTEPS; ++ss) {
            crow[ss] = M::load_perm(cs + 32 * st, ss, lh);
#pragma unroll
            for (int mt = 0; mt < NT; ++mt) {
              gtf[mt][ss] = M::load_perm(Gts + (32 * mt + lr) * PV + 32 * st, ss, lh);
              qtf[mt][ss] = M::load_perm(Qts + (32 * mt + lr) * PV + 32 * st, ss, lh);
            }
          }
          TM::both(s_cur, dp_cur, crow, coef, edge, lo, hi, lh, pb, db);
#pragma unroll
          for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
            for (int mt = 0; mt < NT; ++mt) {
              av[j][mt] = M::mma(gtf[mt][ss], pb[ss], av[j][mt]);
              ak[j][mt] = M::mma(qtf[mt][ss], db[ss], ak[j][mt]);
            }
        }
        s_cur = s_nxt; dp_cur = dp_nxt;
      }
      if (NBUF == 1) FM_SYNC(); else buf ^= 1;
    }
    if (NBUF == 2) FM_SYNC();
  }
  // keys past nk are zero rows: their gradients are discarded by the bounds check
  const float inv_gs = 1.0f / A.gscale;
  fm_store_tokens<TIO, E, DH, QT>(ak, xrow, nullptr, A.sc * inv_gs, reinterpret_cast<float*>(R), A.dk, bh, k0, A.nk, tid);
  fm_store_tokens<TIO, E, DH, QT>(av, xrow, use_state ? vecs + DH : nullptr, inv_gs, reinterpret_cast<float*>(R), A.dv, bh, k0, A.nk,
                                  tid);
}
