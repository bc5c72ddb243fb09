// Token-side kernels: the forward and the three gradients as two kernel shapes.
//
// A workgroup owns QW tokens of one batch*head ("own" tokens: one 32-token tile per
// accumulator column group, QT tiles per wavefront) and streams the tokens of the
// other side past them in stages of KT.  With x_ij = q_i.k_j (q, k pre-multiplied
// by sqrt(1/tau)), f(x) = a0 + a1 x + a2 x^2 and, per query, gh_i = dO_i / g_i,
// c_i = gh_i.o_i:
//
//   k_pv  own = queries:  F_i  = sum_j M_ij f(x_ij) v_j,  g_i = sum_j M_ij f(x_ij)      (forward)
//         own = keys:     dV_j = sum_i M_ij f(x_ij) gh_i
//   k_ds  own = queries:  dQ_i = sum_j dS_ij k_j          dS_ij = M_ij f'(x_ij) (gh_i.v_j - c_i)
//         own = keys:     dK_j = sum_i dS_ij q_i
//
// Stream tokens outside the own token's segment arrive through a moment state
// (fm_readout), those inside it through dense 32x32 tiles; tiles on the causal diagonal
// or at the end of the sequence zero the entries outside their row window.
//
// Replaces calc_masked / calc_unmasked (fastmax_cuda_forward.cu:23-280) and
// calc_gradq/k/v_* (fastmax_cuda_backward.cu:26-491), which walk the tokens serially
// with one thread per feature; the formulas are those of
// fastattention_einops.py:186-322 (forward) and :384-691 (backward).
#pragma once
#include "fm_kernels.h"

enum { FM_OWN_Q = 0, FM_OWN_K = 1 };

template <typename TIO, typename E> struct TokArgs {
  TRef<const TIO> own_io;   // k_pv, own = queries: q in the caller's tensor (multiplied by sc on load)
  const E* own_r;           // otherwise: own tokens, row-major compute-type copy [bh][npad_own][DH]
  const E* own2_r;          // k_ds: second own operand rows (gh for own = queries, v for own = keys)
  const float* cv;          // k_ds: c per query [bh][npad_q], fp32, tokens of every group of 16 in `tperm` order
  const E* xr;              // stream rows that form the scores      [bh][npad_str][DH]
  const E* yr;              // k_ds: stream rows that form gh.v      [bh][npad_str][DH]
  const E* zt;              // stream tokens, transposed             [bh][DH][npad_str]
  const E* zt2;             // k_ds with dV: gh transposed           [bh][DH][npad_str]
  int npad_own, npad_str;
  const E* big; const float* small; int nslots;
  const E* bigb;            // k_ds with dV and order-2 states: the tile-transposed copy of `big` (dV's layout)
  TRef<TIO> out;
  TRef<TIO> out2;           // k_ds with dV: dV
  TRef<float> g;                        // k_pv, own = queries: denominators (bh, n)
  int n_own, n_str, L, nseg, causal, use_state, quad;
  float a0, a1, a2;                     // f(x) = a0 + a1 x + a2 x^2
  float sc;                             // sqrt(1/tau)
  float out_scale;                      // factor on the stored gradient
  float out2_scale;                     // k_ds with dV: factor on dV
  float zscale;                         // factor on the Z of the state (k_ds)
  // k_ds with PREP (own = queries): the kernel makes gh = gscale * dO / g, c = gh . o and q' = sc * q of
  // its own queries itself, from the caller's tensors, and leaves them in w_gh, w_qr (row-major
  // [bh][npad_own][DH]) and w_cv ([bh][npad_own], tile order) for the key-side pass that follows
  TRef<const TIO> own_o, own_do;
  E* w_gh; E* w_qr; float* w_cv;
  // partial maxima of |dO| / |g| ([bh][gnblk], see k_grad_scale) or null: the kernels that form gh multiply it by
  // fm_grad_scale of them, the kernels that store a gradient divide by it
  const float* gpart; int gnblk;
  // Max-norm normalisation folded into the loads (see NormFold).  own_fold: of the own tokens' caller tensor
  // (the kernels that read it: forward, and dQ with PREP); the compute-type copies are made with the factor in.
  // Backward with the normalisation's own Jacobian (bpart != null): the stored gradient is multiplied by
  // out_fold's factor and the workgroup leaves its part of B = sum dy . y (y = normalised rows, taken from
  // the copy `brows` = sc * y) in bpart [bh][blocks]; k_norm_fix applies the rank-one term to one row later.
  NormFold own_fold, out_fold;
  const E* brows; float* bpart;
  // What bf16 rounding takes away from o, [bh][npad_own][DH] halves: o = (the caller's bf16 o) + this.  The forward
  // writes it next to o when its workspace is kept for the backward (out_resid), the backward's preparation adds it
  // back (own_ores) before it forms c = gh . o: c is subtracted from numbers of its own size, gh . v, so the 8 bits
  // of a bf16 o would leave dS with a few bits, and with an error of one sign along a whole row of keys.
  fm_half* out_resid; const fm_half* own_ores;
  // k_ds, own = queries, _Float16: the prefix state is the forward's own layout (slab a = [v][k], see fm_readout's
  // TRA) and its order-2 part is to be counted state_xscale times
  float state_xscale;
};

// eight values as they will read back from the caller's tensor: themselves (fp32) or rounded to bf16
template <typename TIO> FM_DEVICE float fm_as_stored(float v);
template <> FM_DEVICE float fm_as_stored<float>(float v) { return v; }
template <> FM_DEVICE float fm_as_stored<fm_bf16>(float v) { return fm_bf16_to_f32(fm_f32_to_bf16(v)); }
FM_DEVICE void fm_store_resid8(fm_half* p, const float v[8], const float stored[8]) {
  fm_half8 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = fm_half(v[i] - stored[i]);
  *reinterpret_cast<fm_half8*>(p) = r;
}

// Z (fp32, [DH][DH]) -> LDS in the compute type (hi/lo split for _Float16), va/vb -> vecs.
template <typename E, int DH, int QT>
FM_DEVICE void fm_stage_small(const float* sml, E* Zs, float* vecs, int tid, float zscale) {
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
// brows (optional): compute-type rows of the same tokens (row t at brows + (t - brow0) * bpitch: a copy in
// memory, or a tile still in LDS); the workgroup's sum over its stored values times those rows, times bscale,
// goes to *bout (one workgroup-uniform address).
// pitch (floats) of the fp32 staging of fm_store_tokens: rows stay 16-byte aligned
constexpr int fm_store_pitch(int dh) { return dh + 4; }
template <typename TIO, typename E, int DH, int QT>
FM_DEVICE void fm_store_tokens(fm_f32x16 (*acc)[DH / 32], const int* xrow, const float* addvec, float scale, float* Os,
                               TRef<TIO> out, int bh, int row0, int nrows, int tid, const E* brows = nullptr,
                               float bscale = 0.f, float* bout = nullptr, int bpitch = DH, int brow0 = 0) {
  typedef TokCfg<E, DH, QT> C;
  constexpr int OP = fm_store_pitch(DH);                 // rows of the staging 16-byte aligned: four entries per LDS write
  const int lane = tid & 63, lh = lane >> 5;
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int ct = 0; ct < C::NT; ++ct)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int c = 32 * ct + fm_acc_row(4 * g, lh);
        fm_f32x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = scale * (acc[j][ct][4 * g + i] + (addvec ? addvec[c + i] : 0.f));
        *reinterpret_cast<fm_f32x4*>(Os + xrow[j] * OP + c) = w;
      }
  FM_SYNC();
  TIO* ob = out.base(bh);
  float bsum = 0.f;
  for (int c = tid; c < C::QW * (DH / 8); c += FM_THREADS) {
    const int row = c / (DH / 8), col = (c % (DH / 8)) * 8;
    if (row0 + row < nrows) {
      const fm_f32x4 lo = *reinterpret_cast<const fm_f32x4*>(Os + row * OP + col);
      const fm_f32x4 hi = *reinterpret_cast<const fm_f32x4*>(Os + row * OP + col + 4);
      const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      if (brows) {
        const E* br = brows + int64_t(row0 + row - brow0) * bpitch + col;
#pragma unroll
        for (int i = 0; i < 8; ++i) bsum += v[i] * float(br[i]);
      }
      IO<TIO>::st8(ob + int64_t(row0 + row) * out.s_n + col, out.vec != 0, v);
    }
  }
  FM_SYNC();
  if (bout) {
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) bsum += fm_shfl_xor(bsum, m);
    if (lane == 0) Os[tid >> 6] = bsum;
    FM_SYNC();
    if (tid == 0) *bout = bscale * ((Os[0] + Os[1]) + (Os[2] + Os[3]));
    FM_SYNC();
  }
}

// Placement of the blocks of own tokens.  A causal block's work is its dense part (1 .. L/QW
// units of QW x QW tiles, growing with the position inside its segment for queries, shrinking
// for keys) plus the state readout (the same for every block that has a state), so blocks
// differ by up to an order of magnitude, and at B*H = 32, N = 4096 a launch has exactly as
// many workgroups as the chip has slots (two per CU): there is no second wave of workgroups
// to even things out.  Workgroups go round-robin to the 8 XCDs and, inside an XCD, to its
// 32 CUs in launch order, so the XCD-local launch index j is turned into a weight rank
// boustrophedon-wise over rounds of 32: the CU that got the heaviest block of one round gets
// the lightest of the next.  All blocks of one batch*head stay on one XCD (one L2).
FM_DEVICE int fm_snake_rank(int j, int total) {
  const int r = j >> 5, pos = j & 31, base = r << 5;
  if ((r & 1) == 0) return j;
  const int cnt = total - base < 32 ? total - base : 32;
  return base + cnt - 1 - pos;
}

// rank (0 = heaviest) -> block index, for a causal launch with bps blocks per segment.
// Own = queries: the blocks that have a state (segments >= 1) come first, late positions w inside
// the segment before early ones and, for one position, late segments before early ones; then the
// blocks of segment 0, late positions first.  Own = keys: the blocks that have a state (all but the
// last segment), early positions first and, for one position, early segments first; then the last
// segment.  The last segment may be short (wl of bps blocks).  Closed form: a launch over a long
// sequence has hundreds of blocks per batch*head and every wavefront needs its own.
template <int OWN> FM_DEVICE int fm_block_of_rank(int rank, int nblk, int bps) {
  const int nseg = (nblk + bps - 1) / bps;
  const int wl = nblk - (nseg - 1) * bps;              // blocks of the last segment, 1 .. bps
  if (OWN == FM_OWN_Q) {
    if (nseg > 1) {
      const int per_hi = nseg - 2, n_hi = (bps - wl) * per_hi;   // positions the last segment lacks
      if (rank < n_hi) return (nseg - 2 - rank % per_hi) * bps + (bps - 1 - rank / per_hi);
      rank -= n_hi;
      const int per_lo = nseg - 1, n_lo = wl * per_lo;
      if (rank < n_lo) return (nseg - 1 - rank % per_lo) * bps + (wl - 1 - rank / per_lo);
      rank -= n_lo;
    }
    return (nblk < bps ? nblk : bps) - 1 - rank;
  } else {
    const int per = nseg - 1;
    if (rank < bps * per) return (rank % per) * bps + rank / per;
    return per * bps + (rank - bps * per);
  }
}

// Which part of the stream a block of own tokens starting at t0 sees densely, and which state slot.
template <int OWN, int QW, typename A_>
struct TokGeom {
  int unit, bh, t0, seg, slot, sbeg, send;
  bool use_state;
  FM_DEVICE void init(const A_& A) {
    const int nblk = FM_GDIM_X, nbh = FM_GDIM_Y;
    const int id = FM_BID_X + nblk * FM_BID_Y;
    if ((nbh & 7) == 0) {
      const int nb = nbh >> 3;                       // batch*heads per XCD
      const int rank = fm_snake_rank(id >> 3, nblk * nb);
      unit = rank / nb;
      bh = (id & 7) + 8 * (rank % nb);
    } else {
      unit = id % nblk;
      bh = id / nblk;
    }
    // Many segments (a long sequence): the blocks of one segment read the same state, 557 KB at order 2, so
    // they are launched next to each other and run at the same time: the state comes from HBM once and from
    // the L2 for the others (ordered by weight, the blocks of a segment ran far apart and each fetched it
    // again).  With hundreds of blocks per batch*head the dispatcher evens the weights out by itself.
    const bool seg_major = A.causal && A.use_state && A.nseg >= 8;
    const int blk = !A.causal ? unit : seg_major ? (OWN == FM_OWN_Q ? nblk - 1 - unit : unit)
                                                 : fm_block_of_rank<OWN>(unit, nblk, A.L / QW);
    t0 = blk * QW;
    seg = A.causal ? t0 / A.L : 0;
    slot = A.causal ? seg : 0;
    if (OWN == FM_OWN_Q) {
      use_state = A.use_state && (!A.causal || seg > 0);
      sbeg = A.causal ? seg * A.L : 0;
      send = A.causal ? (t0 + QW < A.n_str ? t0 + QW : A.n_str) : (A.use_state ? 0 : A.n_str);
    } else {
      use_state = A.use_state && (!A.causal || seg < A.nseg - 1);
      sbeg = A.causal ? t0 : 0;
      send = A.causal ? ((seg + 1) * A.L < A.n_str ? (seg + 1) * A.L : A.n_str) : (A.use_state ? 0 : A.n_str);
    }
  }
};

// one 32-token stream tile starting at s0 against the own tile starting at lo
template <int OWN> FM_DEVICE bool fm_tile_edge(bool causal, int s0, int lo, int n_str) {
  if (s0 + 31 >= n_str) return true;
  if (!causal) return false;
  return OWN == FM_OWN_Q ? (s0 + 31 > lo) : (s0 < lo + 31);
}
// rows (stream tokens of the tile) that the lane's own token lo + lr may see
template <int OWN> FM_DEVICE void fm_tile_window(bool causal, int s0, int lo, int lr, int n_str, int& wlo, int& whi) {
  wlo = 0;
  whi = n_str - 1 - s0;
  if (causal) {
    const int dgl = lo + lr - s0;
    if (OWN == FM_OWN_Q) { if (dgl < whi) whi = dgl; } else wlo = dgl;
  }
}

// ------------------------------------------------------------------------------
// k_pv: forward (own = queries) and dV (own = keys).  grid (ceil(n_own / QW), bh).
// LDS: va, vb | own rows [QW][PQ] | region (Z, then state slabs); the two dense stages and the
// output staging lie over the own rows and the region once they are spent.
// ------------------------------------------------------------------------------
// QF = 1 (forward of an order-2 problem without states, _Float16): the weights in their completed-square
// form (see TileMath<fm_half>::wq); the host picks it when a2 is of ordinary size.
template <typename TIO, typename E, int DH, int QT, int OWN, int QF = 0>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, (TokCfg<E, DH, QT>::OCC_PV)) k_pv(TokArgs<TIO, E> A) {
  static_assert(!QF || (QT == 1 && OWN == FM_OWN_Q && sizeof(E) == 2), "completed-square weights: forward, one tile per wavefront");
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  typedef TileMath<E> TM;
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, QW = C::QW, PQ = C::PQ, KT = C::KT_PV, PV = C::PV_PV;
  constexpr int STAGE = C::PV_STAGE;
  FM_DYN_SMEM(smem);
  float* vecs = reinterpret_cast<float*>(smem);       // va[DH], vb[DH]
  E* Own = reinterpret_cast<E*>(vecs + 2 * DH);       // [QW][PQ]
  E* R = Own + QW * PQ;
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  TokGeom<OWN, QW, TokArgs<TIO, E> > G;
  G.init(A);
  const int bh = G.bh, t0 = G.t0;
  const bool causal = A.causal != 0;

  // ---- stage the own rows (and the small states) ----
  if (OWN == FM_OWN_Q) {
    RowRegs<TIO, E, QW, DH> rq;
    rq.load(A.own_io.base(bh), A.own_io.s_n, A.own_io.vec != 0, t0, A.n_own, tid);
    rq.store(Own, PQ, tid, A.sc * fm_norm_factor(A.own_fold, bh, lane));
  } else {
    TileRegs<E, QW, DH> ro;
    ro.load(A.own_r + (int64_t(bh) * A.npad_own + t0) * DH, DH, tid);
    ro.store(Own, PQ, tid);
  }
  const float* sml = A.small + (int64_t(bh) * A.nslots + G.slot) * StateDims<DH>::SMALL;
  if (G.use_state) {
    // order 1 has no Z (its coefficient is the order-2 one): only the two vectors are staged
    if (OWN == FM_OWN_Q && A.quad) fm_stage_small<E, DH, QT>(sml, R, vecs, tid, 1.0f);
    else if (tid < 2 * DH) vecs[tid] = sml[DH * DH + tid];
  }
  FM_SYNC();

  int tw[QT], xrow[QT];
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    tw[j] = (j == 0) ? wave : (4 * QT - 1 - wave);   // pair a short and a long causal tile
    xrow[j] = tw[j] * 32 + lr;
  }
  frag of[QT][NKS];
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) of[j][ks] = M::load(Own + xrow[j] * PQ + ks * M::KSTEP + lh * M::KPL);
  fm_f32x16 sseed = fm_zero16();
  if constexpr (QF != 0) {
    // the score products deliver h = 2 a2 s + a1
    const frag t2 = M::splat(CE<E>::from(2.0f * A.a2));
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) of[0][ks] = of[0][ks] * t2;
    sseed = fm_seed16(A.a1);
  }

  fm_f32x16 acc[QT][NT];
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) acc[j][ct] = fm_zero16();
  float gsum[QT];
#pragma unroll
  for (int j = 0; j < QT; ++j) gsum[j] = 0.f;

  if (G.use_state) {
    if (OWN == FM_OWN_Q && A.quad) {
      // denominator: g_i += sum_m q_im (va[m] + sum_l Z[m][l] q_il)
#pragma unroll
      for (int j = 0; j < QT; ++j)
#pragma unroll
        for (int mt = 0; mt < NT; ++mt) {
          const fm_f32x16 y = fm_zy<E, DH, QT>(R, of[j], mt, lr, lh);
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int m = 32 * mt + fm_acc_row(e, lh);
            gsum[j] += (y[e] + vecs[m]) * float(Own[xrow[j] * PQ + m]);
          }
        }
      FM_SYNC();                                       // Z is overwritten by the slabs
    } else if (OWN == FM_OWN_Q) {
      // order 1: g_i += q_i . va, from the half of its row that the lane holds as B fragments (the
      // other half is the other 32 lanes'; the two meet in the epilogue).  No Z was staged, so
      // nothing has to be waited for before the state readout.
#pragma unroll
      for (int j = 0; j < QT; ++j)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
          for (int i = 0; i < M::KPL; ++i) gsum[j] += vecs[ks * M::KSTEP + lh * M::KPL + i] * M::elem(of[j][ks], i);
    }
    const E* state = A.big + (int64_t(bh) * A.nslots + G.slot) * StateDims<DH>::stride(A.quad != 0);
    fm_readout_sym<E, DH, QT, NT>(state, A.quad != 0, Own, xrow, of, R, acc, tid);   // x = y = the own rows, sums symmetric in (a, b)
  } else {
    FM_SYNC();                                         // own rows are overwritten by the dense stages
  }

  // ---- dense tiles over the stream tokens of this segment ----
  if (G.send > G.sbeg) {
    const typename TM::Coef coef = TM::coef(A.a0, A.a1, A.a2);
    // _Float16: the second stream tile is staged row-major too (yr: v rows for the forward, gh rows
    // for dV) and its transposed fragments come from transposing LDS reads; zt is not read then
    constexpr bool TR = M::HAS_TR;
    TileRegs<E, KT, DH> rx, ry;
    TileRegs<E, DH, KT> rz;
    const E* xb = A.xr + int64_t(bh) * A.npad_str * DH;
    const E* yb = TR ? A.yr + int64_t(bh) * A.npad_str * DH : nullptr;
    const E* zb = TR ? nullptr : A.zt + int64_t(bh) * DH * A.npad_str;
    auto fetch = [&](int sx) {                          // global memory -> registers
      rx.load(xb + int64_t(sx) * DH, DH, tid);
      if (TR) ry.load(yb + int64_t(sx) * DH, DH, tid); else rz.load(zb + sx, A.npad_str, tid);
    };
    auto put = [&](int b) {                             // registers -> stage buffer b
      E* Xn = Own + b * STAGE;
      rx.store(Xn, PQ, tid);
      if (TR) ry.store(Xn + KT * PQ, PQ, tid); else rz.store(Xn + KT * PQ, PV, tid);
    };
    // Stages are walked so that all blocks of a batch*head start at the same end of the stream
    // (queries start at the first key of the segment, keys at its last query): blocks that run at
    // the same time then read the same tiles at about the same time and share them in the L2.
    const int nst = (G.send - G.sbeg + KT - 1) / KT;
    const int s_first = OWN == FM_OWN_Q ? G.sbeg : G.sbeg + KT * (nst - 1);
    const int s_step = OWN == FM_OWN_Q ? KT : -KT;
    // Two stage buffers.  The tiles of stage i+1 travel global memory -> registers during stage i-1
    // and registers -> LDS in the middle of stage i (between the two groups of matrix products),
    // so the only thing left at the top of a stage is the barrier.
    auto more = [&](int sx) { return OWN == FM_OWN_Q ? (sx < G.send) : (sx >= G.sbeg); };
    fetch(s_first);
    put(0);
    if (more(s_first + s_step)) fetch(s_first + s_step);
    int buf = 0;
    for (int s0 = s_first; more(s0); s0 += s_step) {
      E* Xs = Own + buf * STAGE;                        // the own rows and the slabs are spent
      E* Zt = Xs + KT * PQ;
      FM_SYNC();
      // One code path for every tile: the products always run, and a tile that touches the mask
      // or the end of the sequence (a wavefront-uniform test) zeroes the entries outside its row
      // window before they are used; a tile wholly outside the mask has an empty window.
#pragma unroll
      for (int st = 0; st < KT / 32; ++st) {
        if (QT == 1) { FM_SCHED_MFMA_DS(0); }
        fm_f32x16 s[QT];
#pragma unroll
        for (int j = 0; j < QT; ++j) s[j] = QF ? sseed : fm_zero16();
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const frag xf = M::load(Xs + (32 * st + lr) * PQ + ks * M::KSTEP + lh * M::KPL);
#pragma unroll
          for (int j = 0; j < QT; ++j) s[j] = M::mma(xf, of[j][ks], s[j]);
        }
        frag zf[NT][M::ACC_KSTEPS];
#pragma unroll
        for (int ct = 0; ct < NT; ++ct)
#pragma unroll
          for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
            zf[ct][ss] = TR ? M::load_tr(Zt, PQ, 32 * st + 16 * ss, 32 * ct, lane)
                            : M::load_perm(Zt + (32 * ct + lr) * PV + 32 * st, ss, lh);
        if (st == KT / 32 - 1) {
          // next stage: registers -> the other buffer (its readers finished before this stage's
          // barrier), then the stage after it: global memory -> registers.  No branch (see k_ds): past the last
          // stage the registers go where nobody reads and the current stage is loaded once more.
          const int sn = s0 + s_step, sf = more(sn) && more(sn + s_step) ? sn + s_step : s0;
          put(buf ^ 1);
          fetch(sf);
        }
#pragma unroll
        for (int j = 0; j < QT; ++j) {
          const int ss0 = s0 + 32 * st, lo = t0 + tw[j] * 32;
          // two tiles per wavefront: skip the second half of tile pairs wholly outside the mask (see k_ds)
          if (QT == 2 && causal && (OWN == FM_OWN_Q ? (ss0 > lo + 31) : (ss0 + 31 < lo))) continue;
          const bool edge = fm_tile_edge<OWN>(causal, ss0, lo, A.n_str);
          int wlo, whi;
          fm_tile_window<OWN>(causal, ss0, lo, lr, A.n_str, wlo, whi);
          frag pb[M::ACC_KSTEPS];
          float gs;
          if constexpr (QF != 0) gs = TM::wq(s[j], TM::pair(4.0f * A.a0 * A.a2 - A.a1 * A.a1), edge, wlo, whi, lh, pb);
          else gs = TM::fwd(s[j], coef, edge, wlo, whi, lh, pb);
          if (OWN == FM_OWN_Q) gsum[j] += gs;
#pragma unroll
          for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) acc[j][ct] = M::mma(zf[ct][ss], pb[ss], acc[j][ct]);
        }
      }
      buf ^= 1;
    }
    FM_SYNC();
  }

  // ---- epilogue, staged through LDS for coalesced stores ----
  float* Os = reinterpret_cast<float*>(Own);           // [QW][fm_store_pitch]
  constexpr int OP = fm_store_pitch(DH);
  if (OWN == FM_OWN_Q) {
    // o = (F + vb) / g
    const float cnt = causal ? float(G.sbeg) : float(A.n_str);   // keys covered by the state
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      float gt = gsum[j] + fm_shfl_xor(gsum[j], 32);
      if (G.use_state) gt += A.a0 * cnt;
      const float ginv = 1.0f / gt;
      if (QF) gt *= 1.0f / (4.0f * A.a2);              // the constant taken out of the weights (o does not see it)
#pragma unroll
      for (int ct = 0; ct < NT; ++ct)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int c = 32 * ct + fm_acc_row(4 * g4, lh);
          fm_f32x4 w;
#pragma unroll
          for (int i = 0; i < 4; ++i) w[i] = (acc[j][ct][4 * g4 + i] + (G.use_state ? vecs[DH + c + i] : 0.f)) * ginv;
          *reinterpret_cast<fm_f32x4*>(Os + xrow[j] * OP + c) = w;
        }
      const int qi = t0 + xrow[j];
      if (lh == 0 && qi < A.n_own) A.g.base(bh)[int64_t(qi) * A.g.s_n] = gt;
    }
    FM_SYNC();
    TIO* ob = A.out.base(bh);
    for (int c = tid; c < QW * (DH / 8); c += FM_THREADS) {
      const int row = c / (DH / 8), col = (c % (DH / 8)) * 8;
      if (t0 + row < A.n_own) {
        const fm_f32x4 lo = *reinterpret_cast<const fm_f32x4*>(Os + row * OP + col);
        const fm_f32x4 hi = *reinterpret_cast<const fm_f32x4*>(Os + row * OP + col + 4);
        const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        IO<TIO>::st8(ob + int64_t(t0 + row) * A.out.s_n + col, A.out.vec != 0, v);
        if (A.out_resid) {
          float sv[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) sv[i] = fm_as_stored<TIO>(v[i]);
          fm_store_resid8(A.out_resid + (int64_t(bh) * A.npad_own + t0 + row) * DH + col, v, sv);
        }
      }
    }
  } else {
    // dV = (sums + vb) * out_scale; keys past n_own are discarded by the bounds check
    const float gsc = fm_grad_scale(A.gpart ? A.gpart + int64_t(bh) * A.gnblk : nullptr, A.gnblk, lane);
    fm_store_tokens<TIO, E, DH, QT>(acc, xrow, G.use_state ? vecs + DH : nullptr, A.out_scale / gsc, Os, A.out, bh, t0,
                                    A.n_own, tid);
  }
}

// ------------------------------------------------------------------------------
// Order-2 suffix state read once for dK and dV of the own keys (one 32-token tile per wavefront).  With
// U[a][c][b] = a2 sum_i q'_a gh_c q'_b (the transposed-tile copy of the state, slab a = rows c, columns b):
//   Y_a[c] = sum_b U[a][c][b] k'_b            8 matrix instructions per slab, B fragments = the key's own rows
//   dV[c] += k'_a Y_a[c]                      the accumulator entries of the lane, fp32
//   dK[a]  = 2 sum_c v_c Y_a[c]               v in accumulator layout; the two halves of a wavefront hold 32 values of c
//                                             each and meet through one cross-lane add; the sum goes to dks[token][a]
// which takes 8 matrix instructions per slab and tile where the two separate readouts take 8 + 5, no Khatri-Rao
// products, and one staging of the state instead of two.
// slab: two buffers of DH * PS elements; dks: [QW][DH + 1] floats, rows of the wavefront's own tokens only (no barrier
// between its writes here and the reads of the same wavefront later).  All 256 threads must call this.
// ------------------------------------------------------------------------------
template <typename E, int DH>
FM_DEVICE void fm_readout_kv(const E* FM_RESTRICT state2, const E* xs, int xrow, const typename Mma<E>::frag* kf,
                             const float (*vacc)[16], E* slab, float* dks, fm_f32x16* av, int tid) {
  typedef TokCfg<E, DH, 1> C;
  typedef Mma<E> M;
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, PS = C::PS;
  constexpr int SLAB1 = DH * PS;
  const int lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int lane_off = lr * PS + lh * M::KPL;
  TileRegs<E, DH, DH> regs;
  regs.load(state2, DH, tid);
  int buf = 0;
  float ka = float(xs[xrow * C::PQ]);
  for (int a = 0; a < DH; ++a) {
    E* sb = slab + buf * SLAB1;
    regs.store(sb, PS, tid);
    FM_SYNC();
    const int an = a + 1 < DH ? a + 1 : a;
    if (a + 1 < DH) regs.load(state2 + int64_t(a + 1) * DH * DH, DH, tid);
    const float kan = float(xs[xrow * C::PQ + an]);
    frag fa[NT][NKS];
#pragma unroll
    for (int ct = 0; ct < NT; ++ct)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) fa[ct][ks] = M::load(sb + lane_off + (32 * ct) * PS + ks * M::KSTEP);
    float dot = 0.f;
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
      fm_f32x16 y = fm_zero16();
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) y = M::mma(fa[ct][ks], kf[ks], y);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        av[ct][e] += ka * y[e];
        dot += vacc[ct][e] * y[e];
      }
    }
    dot += fm_shfl_xor(dot, 32);
    if (lh == 0) dks[xrow * (DH + 1) + a] = 2.0f * dot;
    ka = kan;
    buf ^= 1;
  }
  FM_SYNC();
}

// ------------------------------------------------------------------------------
// k_ds: dQ (own = queries) and dK (own = keys).  grid (ceil(n_own / QW), bh).
// LDS: va, vb | own rows [QW][PQ] | region (Z, then state slabs); the dense stages
// (stream rows for the scores, stream rows for gh.v, stream transposed, c values)
// and the output staging lie over the own rows and the region once they are spent.
// DV = 1 (own = keys, sequences of one segment): the same pass also forms dV from the
// score tiles it already has, P = f(S), dV^T += gh^T P, which saves the four score
// products per tile that a separate k_pv launch would repeat.
// ------------------------------------------------------------------------------
// QF = 1 (order 2 without states, _Float16): completed-square weights and seeded accumulators (see
// TileMath<fm_half>::dsq / bothq); the host picks it when a2 is of ordinary size.
// STR = 1 (own = queries, _Float16, two tiles per wavefront): the prefix state is the forward's own layout and is
// read out transposed (see fm_readout, TRA); the fragments of the dense tiles are fetched behind that readout, so that
// the kernel holds 64 registers fewer across it.
template <typename TIO, typename E, int DH, int QT, int OWN, int DV, int PREP, int QF = 0, int STR = 0>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, (DV ? TokCfg<E, DH, QT>::OCC_DV : TokCfg<E, DH, QT>::OCC_DS)) k_ds(TokArgs<TIO, E> A) {
  static_assert(!STR || (OWN == FM_OWN_Q && sizeof(E) == 2 && !PREP && !QF && !DV), "the transposed readout is dQ's, on _Float16");
  static_assert(!QF || (QT == 1 && sizeof(E) == 2 && (DV != 0 || OWN == FM_OWN_Q)), "completed-square weights: dQ, or dK with dV, one tile per wavefront");
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  typedef TileMath<E> TM;
  typedef typename M::frag frag;
  constexpr int NT = C::NT, NKS = C::NKS, QW = C::QW, PQ = C::PQ;
  constexpr int KT = DV ? C::KT_DV : C::KT_DS, PV = DV ? C::PV_DV : C::PV_DS;
  constexpr int NBUF = C::DS_NBUF;
  constexpr int STAGE = DV ? C::DV_STAGE : C::DS_STAGE;
  // _Float16: the transposed stream tiles (zt = xr^T, zt2 = yr^T) are not staged; their fragments are
  // read out of the staged row tiles with transposing LDS reads (a third to a half fewer bytes per
  // stage, and nobody has to write the transposed copies).  zt and zt2 are not read then.
  constexpr bool TR = M::HAS_TR;
  FM_DYN_SMEM(smem);
  float* vecs = reinterpret_cast<float*>(smem);
  E* Own = reinterpret_cast<E*>(vecs + 2 * DH);       // [QW][PQ]
  E* R = Own + QW * PQ;
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  TokGeom<OWN, QW, TokArgs<TIO, E> > G;
  G.init(A);
  const int bh = G.bh, t0 = G.t0;
  const bool causal = A.causal != 0;
  const float gsc = fm_grad_scale(A.gpart ? A.gpart + int64_t(bh) * A.gnblk : nullptr, A.gnblk, lane);
  const float ginv_sc = 1.0f / gsc;

  if (PREP) {
    // own queries straight from the caller's q, o, dO and g (four threads per token, 64 tokens per
    // pass): q' rows -> Own, gh rows -> R, c behind them; the same values go to the workspace copies
    // the key-side pass streams.  Rows past the end are zeros.  Replaces div_grad_output
    // (fastmax_cuda_backward.cu:494-501) and the "grad * o" row sums of fastattention_einops.py:405-407.
    constexpr int EPT = DH / 4;
    static_assert(!PREP || (OWN == FM_OWN_Q && QT == 1), "the fused preparation is for one query tile per wavefront");
    // PREP = 2: A.own_ores is given (the forward kept what bf16 rounding took from o)
    float* cl = reinterpret_cast<float*>(R + QW * PQ);   // c per own query, behind the gh rows
    const int part = tid & 3, d0 = part * EPT;
    constexpr int NH = QW / 64;
    const float qsc = A.sc * fm_norm_factor(A.own_fold, bh, lane);
    float ra[NH][EPT], rb[NH][EPT], rc[NH][EPT], gi[NH];
    fm_half8 rr[NH][EPT / 8];
    // every load of the block is issued before the first result is used
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      const int row = t0 + 64 * h + (tid >> 2);
      if (row < A.n_own) {
        gi[h] = A.g.base(bh)[int64_t(row) * A.g.s_n];
#pragma unroll
        for (int j = 0; j < EPT; j += 8) {
          IO<TIO>::ld8(A.own_do.base(bh) + int64_t(row) * A.own_do.s_n + d0 + j, A.own_do.vec != 0, &ra[h][j]);
          IO<TIO>::ld8(A.own_o.base(bh) + int64_t(row) * A.own_o.s_n + d0 + j, A.own_o.vec != 0, &rb[h][j]);
          IO<TIO>::ld8(A.own_io.base(bh) + int64_t(row) * A.own_io.s_n + d0 + j, A.own_io.vec != 0, &rc[h][j]);
          if (PREP == 2) rr[h][j / 8] = *reinterpret_cast<const fm_half8*>(A.own_ores + (int64_t(bh) * A.npad_own + row) * DH + d0 + j);
        }
      } else {
        gi[h] = 1.0f;
#pragma unroll
        for (int j = 0; j < EPT; ++j) { ra[h][j] = 0.f; rb[h][j] = 0.f; rc[h][j] = 0.f; }
#pragma unroll
        for (int j = 0; j < EPT / 8; ++j) rr[h][j] = Mma<fm_half>::splat(fm_half(0.f));
      }
    }
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      const int tok = 64 * h + (tid >> 2), row = t0 + tok;
      const float ginv = gsc / gi[h];
      float vg[EPT], vq[EPT];
      float csum = 0.f;
#pragma unroll
      for (int j = 0; j < EPT; ++j) {
        vg[j] = ra[h][j] * ginv;
        csum += vg[j] * (PREP == 2 ? rb[h][j] + float(rr[h][j / 8][j % 8]) : rb[h][j]);   // PREP = 2: o = bf16 o + what its rounding took
        vq[j] = rc[h][j] * qsc;
      }
      csum += fm_shfl_xor(csum, 1);
      csum += fm_shfl_xor(csum, 2);
      if (part == 0) {
        A.w_cv[int64_t(bh) * A.npad_own + t0 + 64 * h + M::tperm(tid >> 2)] = csum;
        cl[tok] = csum;
      }
      E* ghrow = A.w_gh + (int64_t(bh) * A.npad_own + row) * DH + d0;
      E* qrrow = A.w_qr + (int64_t(bh) * A.npad_own + row) * DH + d0;
#pragma unroll
      for (int j = 0; j < EPT; j += 8) {
        CE<E>::st8(ghrow + j, &vg[j]); CE<E>::st8(qrrow + j, &vq[j]);
        CE<E>::st8(R + tok * PQ + d0 + j, &vg[j]); CE<E>::st8(Own + tok * PQ + d0 + j, &vq[j]);
      }
    }
  } else {
    TileRegs<E, QW, DH> ro;
    ro.load(A.own_r + (int64_t(bh) * A.npad_own + t0) * DH, DH, tid);
    ro.store(Own, PQ, tid);
  }
  if (G.use_state) {
    const float* sml = A.small + (int64_t(bh) * A.nslots + G.slot) * StateDims<DH>::SMALL;
    if (A.quad) fm_stage_small<E, DH, QT>(sml, R, vecs, tid, A.zscale);
    else if (tid < 2 * DH) vecs[tid] = sml[DH * DH + tid];   // order 1 has no Z
  }
  FM_SYNC();

  int tw[QT], xrow[QT];
  float ci[QT];                                        // own = queries: c of the lane's query
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    tw[j] = (j == 0) ? wave : (4 * QT - 1 - wave);
    xrow[j] = tw[j] * 32 + lr;
    ci[j] = (OWN == FM_OWN_Q) ? (PREP ? reinterpret_cast<const float*>(R + QW * PQ)[xrow[j]]
                                      : A.cv[int64_t(bh) * A.npad_own + t0 + M::tperm(xrow[j])]) : 1.0f;
  }
  frag of[QT][NKS], of2[QT][NKS];
  auto load_of = [&]() FM_ALWAYS_INLINE {
#pragma unroll
    for (int j = 0; j < QT; ++j)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) of[j][ks] = M::load(Own + xrow[j] * PQ + ks * M::KSTEP + lh * M::KPL);
  };
  auto load_of2 = [&]() FM_ALWAYS_INLINE {
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      const E* o2 = PREP ? R + xrow[j] * PQ + lh * M::KPL
                         : A.own2_r + (int64_t(bh) * A.npad_own + t0 + xrow[j]) * DH + lh * M::KPL;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) of2[j][ks] = M::load(o2 + ks * M::KSTEP);
    }
  };
  // LATE2: the second set is fetched where it is first needed (behind or late in the state readout), not held across it
  constexpr bool LATE2 = STR != 0 || (DV != 0 && OWN == FM_OWN_K && QT == 1 && sizeof(E) == 2 && !QF);
  if constexpr (LATE2) load_of();
  else {
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      const E* o2 = PREP ? R + xrow[j] * PQ + lh * M::KPL
                         : A.own2_r + (int64_t(bh) * A.npad_own + t0 + xrow[j]) * DH + lh * M::KPL;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        of[j][ks] = M::load(Own + xrow[j] * PQ + ks * M::KSTEP + lh * M::KPL);
        of2[j][ks] = M::load(o2 + ks * M::KSTEP);
      }
    }
  }
  fm_f32x16 sseed = fm_zero16(), dpseed = fm_zero16();
  if constexpr (QF != 0) {
    // the score products deliver h = 2 a2 s + a1; the gh.v products start from -c (own = queries: the lane's own c)
    const frag t2 = M::splat(CE<E>::from(2.0f * A.a2));
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) of[0][ks] = of[0][ks] * t2;
    sseed = fm_seed16(A.a1);
    if (OWN == FM_OWN_Q) dpseed = fm_seed16(-ci[0]);
  }
  fm_f32x16 acc[QT][NT], av[DV ? QT : 1][NT];
#pragma unroll
  for (int j = 0; j < QT; ++j)
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) acc[j][mt] = fm_zero16();
#pragma unroll
  for (int j = 0; j < (DV ? QT : 1); ++j)
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) av[j][mt] = fm_zero16();

  if (G.use_state) {
    // - c * (va[m] + sum_l Z[m][l] own_l)   (c = c_i for own = queries; folded into Z and va for own = keys)
#pragma unroll
    for (int j = 0; j < QT; ++j)
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) {
        const fm_f32x16 y = A.quad ? fm_zy<E, DH, QT>(R, of[j], mt, lr, lh) : fm_zero16();
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][mt][e] = -ci[j] * (y[e] + vecs[32 * mt + fm_acc_row(e, lh)]);
      }
    FM_SYNC();                                         // Z is overwritten by the slabs
    const E* state = A.big + (int64_t(bh) * A.nslots + G.slot) * StateDims<DH>::stride(A.quad != 0);
    if constexpr (DV != 0 && QT == 1 && sizeof(E) == 2) {
      // dK and dV from one pass over the order-2 state (the host launches this instantiation with states only for
      // order 2); then the two order-1 slabs, each in its own layout, staged side by side
      const E* state2 = A.bigb + (int64_t(bh) * A.nslots + G.slot) * StateDims<DH>::stride(true);
      float* dks = reinterpret_cast<float*>(R + 2 * C::SLAB);
      float vacc[NT][16];
      {
        const E* vrow = A.own2_r + (int64_t(bh) * A.npad_own + t0 + xrow[0]) * DH;
#pragma unroll
        for (int ct = 0; ct < NT; ++ct)
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            struct alignas(8) Four { E v[4]; };
            const Four f = *reinterpret_cast<const Four*>(vrow + 32 * ct + fm_acc_row(4 * g4, lh));
#pragma unroll
            for (int u = 0; u < 4; ++u) vacc[ct][4 * g4 + u] = float(f.v[u]);
          }
      }
      fm_readout_kv<E, DH>(state2, Own, xrow[0], of[0], vacc, R, dks, av[0], tid);
      load_of2();
      {
        TileRegs<E, DH, DH> s1, s1b;
        s1.load(state + int64_t(DH) * DH * DH, DH, tid);
        s1b.load(state2 + int64_t(DH) * DH * DH, DH, tid);
        s1.store(R, C::PS, tid);
        s1b.store(R + C::SLAB, C::PS, tid);
        FM_SYNC();
        const int lane_off = lr * C::PS + lh * M::KPL;
#pragma unroll
        for (int mt = 0; mt < NT; ++mt) {
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            acc[0][mt] = M::mma(M::load(R + lane_off + (32 * mt) * C::PS + ks * M::KSTEP), of2[0][ks], acc[0][mt]);
            av[0][mt] = M::mma(M::load(R + C::SLAB + lane_off + (32 * mt) * C::PS + ks * M::KSTEP), of[0][ks], av[0][mt]);
          }
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[0][mt][e] += dks[xrow[0] * (DH + 1) + 32 * mt + fm_acc_row(e, lh)];
        }
        FM_SYNC();                                     // the slabs and dks are overwritten by the dense stages
      }
    } else {
      if constexpr (STR != 0) {
        // gh of the own queries in the k order of the transposing reads
        frag ofp[QT][NKS];
#pragma unroll
        for (int j = 0; j < QT; ++j) {
          const E* o2 = A.own2_r + (int64_t(bh) * A.npad_own + t0 + xrow[j]) * DH;
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) ofp[j][ks] = M::load_nat_perm(o2, ks, lh);
        }
        fm_readout<E, DH, QT, NT, true>(state, A.quad != 0, Own, xrow, ofp, R, acc, tid, A.state_xscale);
        load_of(); load_of2();                         // the own rows are still in LDS (fm_readout ends on a barrier)
        FM_SYNC();                                     // ... and are overwritten by the dense stages
      } else {
        fm_readout<E, DH, QT, NT>(state, A.quad != 0, Own, xrow, of2, R, acc, tid);
      }
    }
  } else {
    if (LATE2) load_of2();                             // (a workgroup without a state: no readout)
    FM_SYNC();                                         // own rows are overwritten by the dense stages
  }

  if (G.send > G.sbeg) {
    const typename TM::Coef coef = TM::coef(A.a0, A.a1, A.a2);
    const E* xb = A.xr + int64_t(bh) * A.npad_str * DH;
    const E* yb = A.yr + int64_t(bh) * A.npad_str * DH;
    const E* zb = A.zt + int64_t(bh) * DH * A.npad_str;
    const float* cvb = A.cv + int64_t(bh) * A.npad_str;   // own = keys: c of the streamed queries
    const E* z2b = DV ? A.zt2 + int64_t(bh) * DH * A.npad_str : nullptr;
    // stage order: see k_pv
    const int nst = (G.send - G.sbeg + KT - 1) / KT;
    const int s_first = OWN == FM_OWN_Q ? G.sbeg : G.sbeg + KT * (nst - 1);
    const int s_step = OWN == FM_OWN_Q ? KT : -KT;
    TileRegs<E, KT, DH> rx, ry;
    TileRegs<E, DH, KT> rz, rz2;
    float creg = 0.f;
    auto more = [&](int sx) { return OWN == FM_OWN_Q ? (sx < G.send) : (sx >= G.sbeg); };
    auto fetch = [&](int sx) {                          // global memory -> registers
      rx.load(xb + int64_t(sx) * DH, DH, tid);
      ry.load(yb + int64_t(sx) * DH, DH, tid);
      if (!TR) rz.load(zb + sx, A.npad_str, tid);
      if (DV && !TR) rz2.load(z2b + sx, A.npad_str, tid);
      // c is staged as -c in fp32, tokens in their natural order (the copy holds them in `tperm` order).
      // Every thread takes part (the threads past KT repeat the first ones): no branch in the stage loop.
      if (OWN == FM_OWN_K) creg = cvb[sx + M::tperm(tid % KT)];
    };
    auto put = [&](int b) {                             // registers -> stage buffer b
      E* Xn = Own + b * STAGE; E* Yn = Xn + KT * PQ; E* Zn = Yn + KT * PQ; E* cn = Zn + (TR ? 0 : DH * PV);
      rx.store(Xn, PQ, tid); ry.store(Yn, PQ, tid);
      if (!TR) rz.store(Zn, PV, tid);
      if (DV && !TR) rz2.store(cn + (sizeof(E) == 2 ? 2 : 1) * KT, PV, tid);
      if (OWN == FM_OWN_K) reinterpret_cast<float*>(cn)[tid % KT] = -creg;
    };
    // Two buffers: the tiles of stage i+1 travel global memory -> registers during stage i-1 and
    // registers -> LDS in the middle of stage i (see k_pv).  One buffer (fp32): both at the top.
    fetch(s_first);
    if (NBUF == 2) {
      put(0);
      if (more(s_first + s_step)) fetch(s_first + s_step);
    }
    int buf = 0;
    for (int s0 = s_first; more(s0); s0 += s_step) {
      E* Xs = Own + buf * STAGE; E* Ys = Xs + KT * PQ; E* Zt = Ys + KT * PQ; E* cs = Zt + (TR ? 0 : DH * PV);
      E* Zt2 = cs + (sizeof(E) == 2 ? 2 : 1) * KT;        // behind the KT floats of -c
      if (NBUF == 1) put(0);
      FM_SYNC();
      if (NBUF == 1 && more(s0 + s_step)) fetch(s0 + s_step);
      // One code path for every tile (see k_pv).  The score fragments and the transposed fragments
      // serve all own tiles of the wavefront; gh.v is formed per own tile.
#pragma unroll
      for (int st = 0; st < KT / 32; ++st) {
        if (QT == 1) { FM_SCHED_MFMA_DS(DV ? 0 : 1); }   // two tiles per wavefront: measured slower with it
        fm_f32x16 s[QT];
#pragma unroll
        for (int j = 0; j < QT; ++j) s[j] = QF ? sseed : fm_zero16();
        // One tile per wavefront: the score products and the gh.v products are two chains of dependent matrix
        // instructions that do not depend on each other; issued in turn, each hides the other's latency.
        fm_f32x16 dp1 = fm_zero16();
        if constexpr (QT == 1) {
          if constexpr (QF != 0) {
            if (OWN == FM_OWN_Q) dp1 = dpseed;
            else {
              // -c of the tile's 32 queries, the lane's 16 accumulator rows: four 16-byte reads
              const float* cf = reinterpret_cast<const float*>(cs) + 32 * st + 4 * lh;
#pragma unroll
              for (int gq = 0; gq < 4; ++gq) {
                const fm_f32x4 t = *reinterpret_cast<const fm_f32x4*>(cf + 8 * gq);
                dp1[4 * gq] = t[0]; dp1[4 * gq + 1] = t[1]; dp1[4 * gq + 2] = t[2]; dp1[4 * gq + 3] = t[3];
              }
            }
          }
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            const frag xf = M::load(Xs + (32 * st + lr) * PQ + ks * M::KSTEP + lh * M::KPL);
            const frag yf = M::load(Ys + (32 * st + lr) * PQ + ks * M::KSTEP + lh * M::KPL);
            s[0] = M::mma(xf, of[0][ks], s[0]);
            dp1 = M::mma(yf, of2[0][ks], dp1);
          }
        } else {
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            const frag xf = M::load(Xs + (32 * st + lr) * PQ + ks * M::KSTEP + lh * M::KPL);
#pragma unroll
            for (int j = 0; j < QT; ++j) s[j] = M::mma(xf, of[j][ks], s[j]);
          }
        }
        frag zf[NT][M::ACC_KSTEPS];
        float negc[16];                                  // own = keys, not seeded: -c of the tile's queries, the lane's 16 accumulator rows
        if (OWN == FM_OWN_K && !QF) {
          const float* cf = reinterpret_cast<const float*>(cs) + 32 * st + 4 * lh;
#pragma unroll
          for (int gq = 0; gq < 4; ++gq) {
            const fm_f32x4 t = *reinterpret_cast<const fm_f32x4*>(cf + 8 * gq);
            negc[4 * gq] = t[0]; negc[4 * gq + 1] = t[1]; negc[4 * gq + 2] = t[2]; negc[4 * gq + 3] = t[3];
          }
        }
#pragma unroll
        for (int ss = 0; ss < M::ACC_KSTEPS; ++ss) {
#pragma unroll
          for (int mt = 0; mt < NT; ++mt)
            zf[mt][ss] = TR ? M::load_tr(Xs, PQ, 32 * st + 16 * ss, 32 * mt, lane)
                            : M::load_perm(Zt + (32 * mt + lr) * PV + 32 * st, ss, lh);
        }
        if (NBUF == 2 && st == KT / 32 - 1) {
          // the next stage's tiles into the other buffer and the loads of the stage after it, without a branch: past
          // the last stage the registers are stored where nobody reads and the current stage is loaded once more
          const int sn = s0 + s_step, sf = more(sn) && more(sn + s_step) ? sn + s_step : s0;
          put(buf ^ 1);
          fetch(sf);
        }
#pragma unroll
        for (int j = 0; j < QT; ++j) {
          const int ss0 = s0 + 32 * st, lo = t0 + tw[j] * 32;
          // two tiles per wavefront (256 own tokens, often a whole segment): a good part of the tile
          // pairs lies wholly outside the mask, and skipping their second half pays for the branch
          if (QT == 2 && causal && (OWN == FM_OWN_Q ? (ss0 > lo + 31) : (ss0 + 31 < lo))) continue;
          const bool edge = fm_tile_edge<OWN>(causal, ss0, lo, A.n_str);
          int wlo, whi;
          fm_tile_window<OWN>(causal, ss0, lo, lr, A.n_str, wlo, whi);
          fm_f32x16 dp = dp1;
          if constexpr (QT > 1) {
            if constexpr (QF != 0) {
              if (OWN == FM_OWN_Q) dp = dpseed;
              else {
                // -c of the tile's 32 queries, the lane's 16 accumulator rows: four 16-byte reads
                const float* cf = reinterpret_cast<const float*>(cs) + 32 * st + 4 * lh;
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                  const fm_f32x4 t = *reinterpret_cast<const fm_f32x4*>(cf + 8 * gq);
                  dp[4 * gq] = t[0]; dp[4 * gq + 1] = t[1]; dp[4 * gq + 2] = t[2]; dp[4 * gq + 3] = t[3];
                }
              }
            }
            const E* yrow = Ys + (32 * st + lr) * PQ + lh * M::KPL + FM_OPAQUE_ZERO();
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) dp = M::mma(M::load(yrow + ks * M::KSTEP), of2[j][ks], dp);
          }
          frag db[M::ACC_KSTEPS], pb[M::ACC_KSTEPS];
          if constexpr (QF != 0) {
            if (DV) TM::bothq(s[j], dp, TM::pair(4.0f * A.a0 * A.a2 - A.a1 * A.a1), edge, wlo, whi, lh, pb, db);
            else TM::dsq(s[j], dp, edge, wlo, whi, lh, db);
          } else if (DV) TM::both(s[j], dp, negc, coef, edge, wlo, whi, lh, pb, db);
          else if (OWN == FM_OWN_Q) TM::dsc(s[j], dp, -ci[j], coef, edge, wlo, whi, lh, db);
          else TM::dsr(s[j], dp, negc, coef, edge, wlo, whi, lh, db);
#pragma unroll
          for (int ss = 0; ss < M::ACC_KSTEPS; ++ss)
#pragma unroll
            for (int mt = 0; mt < NT; ++mt) {
              acc[j][mt] = M::mma(zf[mt][ss], db[ss], acc[j][mt]);
              if (DV)
                av[j][mt] = M::mma(TR ? M::load_tr(Ys, PQ, 32 * st + 16 * ss, 32 * mt, lane)
                                      : M::load_perm(Zt2 + (32 * mt + lr) * PV + 32 * st, ss, lh), pb[ss], av[j][mt]);
            }
        }
      }
      if (NBUF == 1) FM_SYNC(); else buf ^= 1;
    }
    if (NBUF == 2) FM_SYNC();
  }
  {
    // with the normalisation's Jacobian: the stored gradient carries lim / max-norm, and the workgroup's part of
    // B = sum dy . y is left for k_norm_fix (the stored values are fac * dy, the copy's rows sc * y)
    const float fac = A.bpart ? fm_norm_factor(A.out_fold, bh, lane) : 1.0f;
    const E* brows = A.bpart ? (PREP ? A.w_qr : A.brows) + int64_t(bh) * A.npad_own * DH : nullptr;
    float* bout = A.bpart ? A.bpart + int64_t(bh) * ((A.n_own + QW - 1) / QW) + t0 / QW : nullptr;
    fm_store_tokens<TIO, E, DH, QT>(acc, xrow, nullptr, A.out_scale * ginv_sc * fac, reinterpret_cast<float*>(Own), A.out, bh, t0,
                                    A.n_own, tid, brows, fac > 0.f ? 1.0f / (fac * A.sc) : 0.f, bout);
  }
  if (DV)
    fm_store_tokens<TIO, E, DH, QT>(av, xrow, G.use_state ? vecs + DH : nullptr, A.out2_scale * ginv_sc * (QF ? 1.0f / (4.0f * A.a2) : 1.0f),
                                    reinterpret_cast<float*>(Own), A.out2, bh, t0, A.n_own, tid);
}
