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
  const E* gh; const E* ght; const E* qt; const E* kt; const float* cv;   // workspace copies
  int npad_q, npad_k;
  const E* bigq; const float* smallq;      // prefix (k, k, v)
  const E* bigk; const float* smallk;      // suffix (q, q, gh)
  const E* bigv; const float* smallv;      // suffix (q, gh, q)
  int nslots;
  int nq, nk, L, nseg, causal, use_state, quad;
  float a0, c1, c2;
};

// Z (fp32, [DH][DH]) -> LDS in the compute type (hi/lo split for _Float16), va/vb -> vecs.
template <typename E, int DH, int QT>
FM_DEVICE void fm_stage_small(const float* sml, E* Zs, float* vecs, int tid) {
  typedef TokCfg<E, DH, QT> C;
  for (int i = tid; i < DH * DH; i += FM_THREADS) {
    const float z = sml[i];
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
FM_DEVICE void fm_store_tokens(fm_f32x16 (*acc)[DH / 32], const int* xrow, const float* addvec, float* Os,
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
        Os[xrow[j] * (DH + 1) + c] = acc[j][ct][e] + (addvec ? addvec[c] : 0.f);
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
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, QW = C::QW, PQ = C::PQ, KT = C::KT, PV = C::PV;
  constexpr int NBUF = sizeof(E) == 2 ? 2 : 1;
  FM_DYN_SMEM(smem);
  E* Qs = reinterpret_cast<E*>(smem);                 // [QW][PQ]  q rows
  E* Gs = Qs + QW * PQ;                               // [QW][PQ]  gh rows
  float* vecs = reinterpret_cast<float*>(Gs + QW * PQ);
  E* R = reinterpret_cast<E*>(vecs + 2 * DH);         // Z | slabs | dense tiles | output staging
  const int tid = FM_TID_X, wave = tid >> 6, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int bh = FM_BID_Y;
  const int nqb = FM_GDIM_X;
  const int qb = A.causal ? (nqb - 1 - FM_BID_X) : FM_BID_X;
  const int q0 = qb * QW;
  const int seg = A.causal ? q0 / A.L : 0;
  const bool use_state = A.use_state && (!A.causal || seg > 0);
  const int slot = A.causal ? seg : 0;
  const int kbeg = A.causal ? seg * A.L : 0;
  const int kend = A.causal ? (q0 + QW < A.nk ? q0 + QW : A.nk) : (A.use_state ? 0 : A.nk);

  {
    RowRegs<TIO, E, QW, DH> rq;
    rq.load(A.q.p + int64_t(bh) * A.q.s_bh, A.q.s_n, A.q.vec != 0, q0, A.nq, tid);
    rq.store(Qs, PQ, tid);
    TileRegs<E, QW, DH> rg;                            // gh rows are dense [npad_q][DH]
    rg.load(A.gh + (int64_t(bh) * A.npad_q + q0) * DH, DH, tid);
    rg.store(Gs, PQ, tid);
  }
  if (use_state)
    fm_stage_small<E, DH, QT>(A.smallq + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL, R, vecs, tid);
  FM_SYNC();

  int tw[QT], xrow[QT];
  float ci[QT];
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    tw[j] = (j == 0) ? wave : (4 * QT - 1 - wave);
    xrow[j] = tw[j] * 32 + lr;
    ci[j] = A.cv[int64_t(bh) * A.npad_q + q0 + xrow[j]];
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
    constexpr int STAGE = 2 * KT * PQ + DH * PV;       // K rows, V rows, K transposed
    RowRegs<TIO, E, KT, DH> rk, rv;
    TileRegs<E, DH, KT> rkt;
    const TIO* kb = A.k.p + int64_t(bh) * A.k.s_bh;
    const TIO* vb = A.v.p + int64_t(bh) * A.v.s_bh;
    const E* ktb = A.kt + int64_t(bh) * DH * A.npad_k;
    rk.load(kb, A.k.s_n, A.k.vec != 0, kbeg, A.nk, tid);
    rv.load(vb, A.v.s_n, A.v.vec != 0, kbeg, A.nk, tid);
    rkt.load(ktb + kbeg, A.npad_k, tid);
    const float c2x2 = 2.0f * A.c2;
    int buf = 0;
    for (int kt0 = kbeg; kt0 < kend; kt0 += KT) {
      E* Ks = R + buf * STAGE; E* Vs = Ks + KT * PQ; E* Kts = Vs + KT * PQ;
      rk.store(Ks, PQ, tid); rv.store(Vs, PQ, tid); rkt.store(Kts, PV, tid);
      FM_SYNC();
      if (kt0 + KT < kend) {
        rk.load(kb, A.k.s_n, A.k.vec != 0, kt0 + KT, A.nk, tid);
        rv.load(vb, A.v.s_n, A.v.vec != 0, kt0 + KT, A.nk, tid);
        rkt.load(ktb + kt0 + KT, A.npad_k, tid);
      }
#pragma unroll
      for (int st = 0; st < KT / 32; ++st) {
        const int key0 = kt0 + 32 * st;
        if (key0 >= kend) break;
        frag kf[NKS], vf[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          kf[ks] = M::load(Ks + (32 * st + lr) * PQ + ks * M::KSTEP + lh * M::KPL);
          vf[ks] = M::load(Vs + (32 * st + lr) * PQ + ks * M::KSTEP + lh * M::KPL);
        }
#pragma unroll
        for (int j = 0; j < QT; ++j) {
          const int qlo = q0 + tw[j] * 32;
          if (A.causal && key0 > qlo + 31) continue;
          fm_f32x16 s = fm_zero16(), dp = fm_zero16();
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            s = M::mma(kf[ks], qf[j][ks], s);
            dp = M::mma(vf[ks], gf[j][ks], dp);
          }
          const bool edge = (A.causal && key0 + 31 > qlo) || (key0 + 31 >= A.nk);
          const int qi = qlo + lr;
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            float ds = (A.c1 + c2x2 * s[e]) * (dp[e] - ci[j]);
            if (edge) {
              const int t = key0 + fm_acc_row(e, lh);
              if ((A.causal && t > qi) || t >= A.nk) ds = 0.f;
            }
            s[e] = ds;
          }
#pragma unroll
          for (int ss = 0; ss < M::ACC_KSTEPS; ++ss) {
            const frag db = M::from_acc(s, ss);
#pragma unroll
            for (int mt = 0; mt < NT; ++mt)
              acc[j][mt] = M::mma(M::load_perm(Kts + (32 * mt + lr) * PV + 32 * st, ss, lh), db, acc[j][mt]);
          }
        }
      }
      if (NBUF == 1) FM_SYNC(); else buf ^= 1;
    }
    if (NBUF == 2) FM_SYNC();
  }
  fm_store_tokens<TIO, E, DH, QT>(acc, xrow, nullptr, reinterpret_cast<float*>(R), A.dq, bh, q0, A.nq, tid);
}

// ------------------------------------------------------------------------------
// k_dkv: gradients with respect to one block of QW keys/values.  grid (ceil(nk/QW), bh).
// ------------------------------------------------------------------------------
template <typename TIO, typename E, int DH, int QT>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS) k_dkv(BwdArgs<TIO, E> A) {
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, KW = C::QW, PQ = C::PQ, KT = C::KT, PV = C::PV;
  constexpr int NBUF = sizeof(E) == 2 ? 2 : 1;
  FM_DYN_SMEM(smem);
  E* Ks = reinterpret_cast<E*>(smem);                 // [KW][PQ]  k rows
  E* Vs = Ks + KW * PQ;                               // [KW][PQ]  v rows
  float* vecs = reinterpret_cast<float*>(Vs + KW * PQ);   // va (dK), vb (dK, unused), then vb of dV at [2*DH..)
  float* vecv = vecs + 2 * DH;
  E* R = reinterpret_cast<E*>(vecv + 2 * DH);
  const int tid = FM_TID_X, wave = tid >> 6, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int bh = FM_BID_Y;
  const int k0 = FM_BID_X * KW;                        // early key blocks are the heavy ones
  const int seg = A.causal ? k0 / A.L : 0;
  const bool use_state = A.use_state && (!A.causal || seg < A.nseg - 1);
  const int slot = A.causal ? seg : 0;
  const int ibeg = A.causal ? k0 : 0;
  int iend = A.causal ? ((seg + 1) * A.L < A.nq ? (seg + 1) * A.L : A.nq) : (A.use_state ? 0 : A.nq);

  {
    RowRegs<TIO, E, KW, DH> rk;
    rk.load(A.k.p + int64_t(bh) * A.k.s_bh, A.k.s_n, A.k.vec != 0, k0, A.nk, tid);
    rk.store(Ks, PQ, tid);
    rk.load(A.v.p + int64_t(bh) * A.v.s_bh, A.v.s_n, A.v.vec != 0, k0, A.nk, tid);
    rk.store(Vs, PQ, tid);
  }
  if (use_state) {
    fm_stage_small<E, DH, QT>(A.smallk + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL, R, vecs, tid);
    if (tid < DH) vecv[tid] = A.smallv[(int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL + DH * DH + DH + tid];
  }
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
    constexpr int STAGE = 2 * KT * PQ + 2 * DH * PV;   // q rows, gh rows, q transposed, gh transposed
    constexpr int STAGE_PAD = STAGE + (KT * 4 + sizeof(E) - 1) / sizeof(E);   // + c values (fp32)
    RowRegs<TIO, E, KT, DH> rq;
    TileRegs<E, KT, DH> rg;
    TileRegs<E, DH, KT> rqt, rgt;
    const TIO* qb = A.q.p + int64_t(bh) * A.q.s_bh;
    const E* ghb = A.gh + int64_t(bh) * A.npad_q * DH;
    const E* qtb = A.qt + int64_t(bh) * DH * A.npad_q;
    const E* gtb = A.ght + int64_t(bh) * DH * A.npad_q;
    const float* cvb = A.cv + int64_t(bh) * A.npad_q;
    float creg = 0.f;
    rq.load(qb, A.q.s_n, A.q.vec != 0, ibeg, A.nq, tid);
    rg.load(ghb + int64_t(ibeg) * DH, DH, tid);
    rqt.load(qtb + ibeg, A.npad_q, tid);
    rgt.load(gtb + ibeg, A.npad_q, tid);
    if (tid < KT) creg = cvb[ibeg + tid];
    const float c2x2 = 2.0f * A.c2;
    int buf = 0;
    for (int i0 = ibeg; i0 < iend; i0 += KT) {
      E* Qr = R + buf * STAGE_PAD; E* Gr = Qr + KT * PQ; E* Qts = Gr + KT * PQ; E* Gts = Qts + DH * PV;
      float* cs = reinterpret_cast<float*>(Gts + DH * PV);
      rq.store(Qr, PQ, tid); rg.store(Gr, PQ, tid); rqt.store(Qts, PV, tid); rgt.store(Gts, PV, tid);
      if (tid < KT) cs[tid] = creg;
      FM_SYNC();
      if (i0 + KT < iend) {
        rq.load(qb, A.q.s_n, A.q.vec != 0, i0 + KT, A.nq, tid);
        rg.load(ghb + int64_t(i0 + KT) * DH, DH, tid);
        rqt.load(qtb + i0 + KT, A.npad_q, tid);
        rgt.load(gtb + i0 + KT, A.npad_q, tid);
        if (tid < KT) creg = cvb[i0 + KT + tid];
      }
#pragma unroll
      for (int st = 0; st < KT / 32; ++st) {
        const int qi0 = i0 + 32 * st;
        if (qi0 >= iend) break;
        frag qf[NKS], gf[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          qf[ks] = M::load(Qr + (32 * st + lr) * PQ + ks * M::KSTEP + lh * M::KPL);
          gf[ks] = M::load(Gr + (32 * st + lr) * PQ + ks * M::KSTEP + lh * M::KPL);
        }
        float crow[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) crow[e] = cs[32 * st + fm_acc_row(e, lh)];
#pragma unroll
        for (int j = 0; j < QT; ++j) {
          const int klo = k0 + tw[j] * 32;             // first key of this tile
          if (A.causal && qi0 + 31 < klo) continue;    // all these queries precede the keys
          fm_f32x16 s = fm_zero16(), dp = fm_zero16();
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            s = M::mma(qf[ks], kf[j][ks], s);
            dp = M::mma(gf[ks], vf[j][ks], dp);
          }
          const bool edge = (A.causal && qi0 < klo + 31) || (qi0 + 31 >= A.nq);
          const int kj = klo + lr;
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const float x = s[e];
            float pv = A.a0 + x * (A.c1 + A.c2 * x);
            float ds = (A.c1 + c2x2 * x) * (dp[e] - crow[e]);
            if (edge) {
              const int i = qi0 + fm_acc_row(e, lh);
              if ((A.causal && i < kj) || i >= A.nq) { pv = 0.f; ds = 0.f; }
            }
            s[e] = pv;
            dp[e] = ds;
          }
#pragma unroll
          for (int ss = 0; ss < M::ACC_KSTEPS; ++ss) {
            const frag pb = M::from_acc(s, ss);
            const frag db = M::from_acc(dp, ss);
#pragma unroll
            for (int mt = 0; mt < NT; ++mt) {
              av[j][mt] = M::mma(M::load_perm(Gts + (32 * mt + lr) * PV + 32 * st, ss, lh), pb, av[j][mt]);
              ak[j][mt] = M::mma(M::load_perm(Qts + (32 * mt + lr) * PV + 32 * st, ss, lh), db, ak[j][mt]);
            }
          }
        }
      }
      if (NBUF == 1) FM_SYNC(); else buf ^= 1;
    }
    if (NBUF == 2) FM_SYNC();
  }
  // keys past nk are zero rows: their gradients are discarded by the bounds check
  fm_store_tokens<TIO, E, DH, QT>(ak, xrow, nullptr, reinterpret_cast<float*>(R), A.dk, bh, k0, A.nk, tid);
  fm_store_tokens<TIO, E, DH, QT>(av, xrow, use_state ? vecv : nullptr, reinterpret_cast<float*>(R), A.dv, bh, k0, A.nk, tid);
}
