// k_walk_sym: the order-2 state walk held per VALUE column (_Float16, D = 64).
//
// A state is U[c][a][b] = sum_t x_tc k_ta k_tb with x the value-like operand (v for the forward's prefix
// walk, gh for the backward's suffix walk) and k the key-like one (k', q').  For a fixed c it is symmetric in
// (a, b).  A wavefront owns one value column c and keeps its 64 x 64 slice as the three 32 x 32 tiles on and
// above the diagonal: per k-step (16 tokens) it reads the two fragments of the key tile once, uses them as the
// B operand and, multiplied by the value row's fragment (v_pk_mul_f16), as the A operand, and issues 3 matrix
// instructions where a walk that holds its slice per key index issues 4 and stages a second 64-row tile.
// A workgroup owns four consecutive values (grid: DH / 4 workgroups per batch*head), walks the tokens once and
// writes a snapshot at every segment boundary, so the prefix (suffix) scan over segments is implicit.
//
// A fifth wavefront does nothing but store.  On this hardware a wavefront's loads and stores retire through one
// in-order counter, so a wavefront that has just issued the 32 KB of a snapshot cannot use the next tile's loads
// before those stores have reached memory, and at a segment end all 256 workgroups store at once: measured at
// B*H = 16, N = 65536, 0.24 of the 0.61 ms of a walk were spent there.  The four summing wavefronts therefore only
// leave the snapshot (and their parts of the lower-order tile) in LDS; the fifth copies it to memory a slice per
// tile over the next segment (two snapshot buffers), never loads, and so never waits for its own stores.
//
// What it writes per segment slot (the layouts the readers already use):
//   o2    [a][c][b]   = coef2 * U[c][a][b]      slab a = rows c, columns b: the forward's and the key side's layout
//                       (a wavefront's rows: 128 contiguous bytes per a; the four wavefronts' rows lie side by side)
//   o1_vk [c][b]      = coef1 * sum x_c k_b      order-1 slab, value-major   (or null)
//   o1_kv [b][c]      = the same, key-major                                   (or null)
//   small { Z[a][b] = coefz * sum w k_a k_b,  va[a] = coefva * sum w k_a,  vb[c] = coefvb * sum x_c }   fp32
// with w a per-token weight (the backward's c_t = gh_t . o_t; ones when cw is null).  The lower-order sums are
// twelve 32 x 32 tiles (4 order-1, 4 Z, 2 va, 2 vb), dealt to the first twelve workgroups of a batch*head; every
// workgroup stages, besides the key tile and its four value rows, the 32 value rows its tile needs, and inside a
// workgroup each wavefront adds a quarter of the k-steps (the four parts meet in LDS at the end of a segment).
//
// Replaces, like k_build, the running sums of fastmax_cuda_forward.cu:165-276 / fastmax_cuda_backward.cu:268-491
// and the cumsum of materialised outer products of fastattention_einops.py:237-248.
#pragma once
#include "fm_kernels.h"

struct WalkSymArgs {
  const fm_half* kt;        // [bh][DH][npad] key-like operand, transposed
  const fm_half* xt;        // [bh][DH][npad] value-like operand, transposed
  const float* cw;          // [bh][npad] per-token weights of Z and va (same token order as the tiles), or null: ones
  int npad, nseg, L, mode, nslots;
  fm_half* o2;              // [bh][nslots][StateDims::BIG]
  fm_half* o1_vk;           // [bh][nslots][StateDims::BIG], the order-1 slab inside, or null
  fm_half* o1_kv;           // likewise
  float* small;             // [bh][nslots][StateDims::SMALL]
  float coef2, coef1, coefz, coefva, coefvb;
};

template <int DH> struct WalkSymCfg {
  typedef Mma<fm_half> M;
  static constexpr int TT = 128;                       // tokens per tile
  static constexpr int PT = TT + M::PAD;
  static constexpr int XR = 8;                         // rows of the x tile: four values, the weights, ones (two spare)
  static constexpr int ROWS = DH + 32 + XR;            // key tile, the lower-order tile's value rows, x rows
  static constexpr int TILE_E = ROWS * PT;             // elements of one buffer
  static constexpr int SP = DH + M::PAD;               // pitch of the snapshot staging
  static constexpr size_t SNAP_BYTES = size_t(4) * DH * SP * 2;       // one snapshot of the four slices, staged
  static constexpr size_t RED_BYTES = size_t(4) * 16 * 64 * 4;        // the four wavefronts' parts of the lower-order tile
  static constexpr size_t lds_bytes() { return size_t(2) * TILE_E * 2 + 2 * SNAP_BYTES + RED_BYTES; }
  static constexpr int THREADS = FM_THREADS + 64;      // four wavefronts that sum, one that stores
};

template <int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS + 64, 1) k_walk_sym(WalkSymArgs A) {
  static_assert(DH == 64, "two 32-row tiles per feature axis");
  typedef fm_half E;
  typedef Mma<E> M;
  typedef typename M::frag frag;
  typedef WalkSymCfg<DH> C;
  constexpr int TT = C::TT, PT = C::PT, NSTEP = TT / M::KSTEP, NT = DH / 32;
  constexpr int NSMALL = 2 * NT * NT + 2 * NT;
  FM_DYN_SMEM(smem);
  E* const buf0 = reinterpret_cast<E*>(smem);
  E* const buf1 = buf0 + C::TILE_E;
  E* const snap0 = buf1 + C::TILE_E;                                   // two staged snapshots: [wave][a][SP]
  float* const red = reinterpret_cast<float*>(smem + size_t(2) * C::TILE_E * sizeof(E) + 2 * C::SNAP_BYTES);   // [4 waves][16][64 lanes]
  constexpr int SNAP_E = int(C::SNAP_BYTES / sizeof(E));
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  int grp, bh;
  const int G = FM_GDIM_X;
  fm_xcd_map(G, FM_GDIM_Y, grp, bh);
  const int nsteps = (A.mode == FM_WALK_TOTAL) ? 1 : A.nseg - 1;
  if (nsteps <= 0) return;
  const int64_t tb_off = int64_t(bh) * DH * A.npad;
  const int c0 = 4 * grp;
  // the lower-order tile of this workgroup (SMALL_NONE: none; it then computes one nobody stores)
  const int tl = grp < NSMALL ? grp : -1;
  // its A operand: 32 value rows (order 1, vb) or 32 key rows times the weights (Z, va); its B operand: 32 key rows or ones
  int sv0 = 0;                                         // first of the 32 value rows staged for it
  int sa_off, sb_off, sw_off;                          // offsets (elements) inside a buffer
  {
    constexpr int OK = 0, OS = DH * PT, OX = (DH + 32) * PT;
    const int ow = OX + 4 * PT, oone = OX + 5 * PT;
    int pa = OK, pb = oone, pw = oone;
    if (tl >= 0 && tl < NT * NT) { sv0 = 32 * (tl / NT); pa = OS; pb = OK + 32 * (tl % NT) * PT; }
    else if (tl >= NT * NT && tl < 2 * NT * NT) { const int u = tl - NT * NT; pa = OK + 32 * (u / NT) * PT; pb = OK + 32 * (u % NT) * PT; pw = ow; }
    else if (tl >= 2 * NT * NT && tl < 2 * NT * NT + NT) { pa = OK + 32 * (tl - 2 * NT * NT) * PT; pw = ow; }
    else if (tl >= 2 * NT * NT + NT) { sv0 = 32 * (tl - 2 * NT * NT - NT); pa = OS; }
    sa_off = pa + lr * PT + lh * M::KPL;
    sb_off = pb == oone ? oone + lh * M::KPL : pb + lr * PT + lh * M::KPL;
    sw_off = pw + lh * M::KPL;
  }

  // cursors: `cur` the tile being summed, `pf` the tile whose loads are issued next (two tiles ahead)
  struct Cursor { int t, w, tb, te, slot; bool valid; };
  auto advance = [&](Cursor& c) {
    c.t += TT;
    if (c.t >= c.te) {
      c.w += 1;
      if (c.w < nsteps) { fm_walk_step(A.mode, A.nseg, A.L, A.npad, c.w, c.tb, c.te, c.slot); c.t = c.tb; }
      else c.valid = false;
    }
  };
  Cursor cur;
  cur.w = 0; cur.valid = true;
  fm_walk_step(A.mode, A.nseg, A.L, A.npad, 0, cur.tb, cur.te, cur.slot);
  cur.t = cur.tb;
  Cursor pf = cur;

  if (wave == 4) {
    // ---- the storing wavefront: follows the walk tile by tile (same barriers), copies the pending snapshot a slice
    // per tile, and at a segment end takes over the new one: what is left of the old one goes out first, then the
    // lower-order tile (the four parts added in a fixed order)
    constexpr int SP = C::SP;
    constexpr int CH = 4 * DH * (DH / 8);                 // 16-byte chunks of a snapshot
    const int per_tile = (CH * TT / A.L + 63) / 64 * 64;  // chunks per tile: a segment's tiles cover the snapshot
    int pend_lo = CH, pend_snap = 0, pend_slot = 0, nsn = 0;
    // chunk c = a * 32 + w * 8 + j (value of a, wavefront's column w, 16-byte piece j of the row): pend_lo is a multiple
    // of 64, so a lane keeps its (w, j) and steps a by two from one chunk to its next -- one LDS read, one store and
    // two additions per chunk (this wavefront shares its SIMD with a summing one: what it issues, that one waits for)
    static_assert(4 * (DH / 8) == 32, "a lane's chunks differ in a only");
    const int cp_w = (lane / (DH / 8)) % 4, cp_b8 = (lane % (DH / 8)) * 8, cp_a0 = lane / 32;
    auto copy = [&](int upto) {
      const int a = pend_lo / 32 + cp_a0;
      const E* src = snap0 + (pend_snap & 1) * SNAP_E + (cp_w * DH + a) * SP + cp_b8;
      E* dst = A.o2 + (int64_t(bh) * A.nslots + pend_slot) * StateDims<DH>::BIG + int64_t(c0) * DH +
               (int64_t(a) * DH + cp_w) * DH + cp_b8;
      for (int c = pend_lo; c < upto; c += 64) {
        *reinterpret_cast<fm_u32x4*>(dst) = *reinterpret_cast<const fm_u32x4*>(src);
        src += 2 * SP; dst += 2 * DH * DH;
      }
      pend_lo = upto;
    };
    // the lower-order tile of a segment end: the four wavefronts' parts, added in a fixed order, to their places in `slot`
    auto put_small = [&](int slot) {
    if (tl >= 0) {
      struct alignas(8) Four { E v[4]; };
      float v[16];
#pragma unroll
      for (int e = 0; e < 16; ++e)
        v[e] = (red[(0 * 16 + e) * 64 + lane] + red[(1 * 16 + e) * 64 + lane]) + (red[(2 * 16 + e) * 64 + lane] + red[(3 * 16 + e) * 64 + lane]);
      const int64_t so = (int64_t(bh) * A.nslots + slot) * StateDims<DH>::BIG + StateDims<DH>::slab1(true);
      float* ds = A.small + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL;
      if (tl < NT * NT) {
        const int r0 = 32 * (tl / NT), cc = 32 * (tl % NT) + lr;        // rows: values, columns: key features
        if (A.o1_vk) {
          E* d1 = A.o1_vk + so;
#pragma unroll
          for (int e = 0; e < 16; ++e) d1[(r0 + fm_acc_row(e, lh)) * DH + cc] = E(A.coef1 * v[e]);
        }
        if (A.o1_kv) {
          E* d2 = A.o1_kv + so;
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            Four f;
#pragma unroll
            for (int u = 0; u < 4; ++u) f.v[u] = E(A.coef1 * v[4 * g4 + u]);
            *reinterpret_cast<Four*>(d2 + cc * DH + r0 + fm_acc_row(4 * g4, lh)) = f;
          }
        }
      } else if (tl < 2 * NT * NT) {
        const int u = tl - NT * NT;
        float* dz = ds + 32 * (u / NT) * DH + 32 * (u % NT) + lr;
#pragma unroll
        for (int e = 0; e < 16; ++e) dz[fm_acc_row(e, lh) * DH] = A.coefz * v[e];
      } else if (lr == 0) {
        const bool is_va = tl < 2 * NT * NT + NT;
        float* dv = ds + DH * DH + (is_va ? 32 * (tl - 2 * NT * NT) : DH + 32 * (tl - 2 * NT * NT - NT));
        const float cf = is_va ? A.coefva : A.coefvb;
#pragma unroll
        for (int e = 0; e < 16; ++e) dv[fm_acc_row(e, lh)] = cf * v[e];
      }
    }
    };
    FM_SYNC();                                            // the prologue's barrier
    bool red_ready = false; int red_slot = 0;
    while (true) {
      // what the last segment end left: first the lower-order tile (its parts stay in LDS until the next segment end;
      // done here, behind the tile's barrier, the summing wavefronts never wait for it), then this tile's share of the copy
      if (red_ready) { put_small(red_slot); red_ready = false; }
      if (pend_lo < CH) copy(pend_lo + per_tile < CH ? pend_lo + per_tile : CH);
      const bool last = cur.t + TT >= cur.te;
      if (last) {
        FM_SYNC();                                        // the snapshot and the parts of the lower-order tile are in LDS
        if (pend_lo < CH) copy(CH);                       // (a segment shorter than the others: the old snapshot's rest)
        pend_lo = 0; pend_snap = nsn; pend_slot = cur.slot; ++nsn;
        red_ready = true; red_slot = cur.slot;
      }
      advance(cur);
      if (!cur.valid) break;
      FM_SYNC();                                          // the tile's barrier
    }
    if (red_ready) put_small(red_slot);
    if (pend_lo < CH) copy(CH);
    return;
  }

  struct Regs { TileRegs<E, DH, TT> k; TileRegs<E, 32, TT> s; TileRegs<E, 4, TT> x; fm_f32x4 w; };
  constexpr int NK = TileRegs<E, DH, TT>::N, NS = TileRegs<E, 32, TT>::N;
  constexpr int NITEM = NK + NS + 2;
  const float* const cwb = A.cw ? A.cw + int64_t(bh) * A.npad : nullptr;
  const int wl = (tid & 31) * 4;                        // the thread's four weights of a tile
  const float* const dummy_w = A.small + int64_t(bh) * A.nslots * StateDims<DH>::SMALL + wl;
  auto load_item = [&](Regs& R, int t, int it) FM_ALWAYS_INLINE {
    if (it < NK) R.k.load_part(A.kt + tb_off + t, A.npad, tid, it);
    else if (it < NK + NS) R.s.load_part(A.xt + tb_off + int64_t(sv0) * A.npad + t, A.npad, tid, it - NK);
    else if (it == NK + NS) R.x.load_wrapped(A.xt + tb_off + int64_t(c0) * A.npad + t, A.npad, tid);
    else R.w = *reinterpret_cast<const fm_f32x4*>(cwb ? cwb + t + wl : dummy_w);   // no branch: without weights, four floats nobody uses
  };
  auto store_item = [&](const Regs& R, E* nb, int it) FM_ALWAYS_INLINE {
    if (it < NK) R.k.store_part(nb, PT, tid, it);
    else if (it < NK + NS) R.s.store_part(nb + DH * PT, PT, tid, it - NK);
    else if (it == NK + NS) R.x.store_wrapped(nb + (DH + 32) * PT, PT, tid);
    else {
      // the weights as halves into x row 4 (every thread writes: the threads past the first 32 repeat them)
      struct alignas(8) Four { E v[4]; };
      Four f;
#pragma unroll
      for (int i = 0; i < 4; ++i) f.v[i] = cwb ? E(R.w[i]) : E(1.0f);
      *reinterpret_cast<Four*>(nb + (DH + 32 + 4) * PT + wl) = f;
    }
  };
  // x row 5 of both buffers: ones (written once)
  if (tid < 2 * TT) (tid < TT ? buf0 : buf1)[(DH + 32 + 5) * PT + (tid % TT)] = E(1.0f);

  fm_f32x16 acc00 = fm_zero16(), acc01 = fm_zero16(), acc11 = fm_zero16(), sacc = fm_zero16();
  Regs R0, R1;
#pragma unroll
  for (int it = 0; it < NITEM; ++it) load_item(R0, pf.t, it);
  advance(pf);
#pragma unroll
  for (int it = 0; it < NITEM; ++it) store_item(R0, buf0, it);
  {
    const int t = pf.valid ? pf.t : cur.t;
#pragma unroll
    for (int it = 0; it < NITEM; ++it) load_item(R1, t, it);
    if (pf.valid) advance(pf);
  }
  FM_WAIT_GLOBAL_LOADS();
  FM_SYNC();

  // End of a segment, summing wavefronts: the slice (rounded, with its coefficient) goes to the snapshot buffer of this
  // segment's parity and the wavefront's part of the lower-order tile to the reduction scratch; the barrier that
  // follows hands both to the storing wavefront.  The slice is symmetric, so a lane writes the transposed entries:
  // its four consecutive accumulator rows are four consecutive columns of row `lr` (8-byte writes); only the tile
  // above the diagonal also needs its straight entries (2-byte writes).
  auto finish_segment = [&](int nsnap) FM_ALWAYS_INLINE {
#if !defined(FM_HOSTSIM)
    // keeps the copies out of the accumulation registers inside this branch (see k_build)
    asm volatile("" : "+a"(acc00)); asm volatile("" : "+a"(acc01)); asm volatile("" : "+a"(acc11)); asm volatile("" : "+a"(sacc));
#endif
    constexpr int SP = C::SP;
    E* stg = snap0 + (nsnap & 1) * SNAP_E + wave * DH * SP;            // this wavefront's [a][b]
    struct alignas(8) Four { E v[4]; };
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      Four f00, f01, f11;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        f00.v[u] = E(A.coef2 * acc00[4 * g4 + u]);
        f01.v[u] = E(A.coef2 * acc01[4 * g4 + u]);
        f11.v[u] = E(A.coef2 * acc11[4 * g4 + u]);
      }
      const int r = fm_acc_row(4 * g4, lh);
      *reinterpret_cast<Four*>(stg + lr * SP + r) = f00;
      *reinterpret_cast<Four*>(stg + (32 + lr) * SP + r) = f01;
      *reinterpret_cast<Four*>(stg + (32 + lr) * SP + 32 + r) = f11;
#pragma unroll
      for (int u = 0; u < 4; ++u) stg[(r + u) * SP + 32 + lr] = f01.v[u];
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) red[(wave * 16 + e) * 64 + lane] = sacc[e];
    FM_SYNC();
  };

  // One tile: the fragments of a k-step are requested two k-steps ahead of their products; behind the products of
  // every k-step one item of the next tile goes registers -> the other buffer and one item of the tile after it
  // global memory -> registers (see k_build for the measurements behind this shape).
  auto body = [&](const Regs& Rs, Regs& Rf, const E* cb, E* nb) FM_ALWAYS_INLINE {
    const E* kb_ = cb + lr * PT + lh * M::KPL;
    const E* xb_ = cb + (DH + 32) * PT + wave * PT + lh * M::KPL;
    const int tn = pf.valid ? pf.t : cur.t;
    constexpr int AHEAD = 2;
    frag fk[NSTEP][NT], fx[NSTEP];
    auto frags = [&](int u) FM_ALWAYS_INLINE {
      fx[u] = M::load(xb_ + u * M::KSTEP);
#pragma unroll
      for (int j = 0; j < NT; ++j) fk[u][j] = M::load(kb_ + 32 * j * PT + u * M::KSTEP);
    };
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) frags(u);
    constexpr int SK = NSTEP / 4;                        // k-steps of the lower-order tile this wavefront takes: wave, wave + 4
    frag sa[SK], sb[SK];
#pragma unroll
    for (int u = 0; u < NSTEP; ++u) {
#if !defined(FM_HOSTSIM)
      __builtin_amdgcn_sched_barrier(0);
#endif
      if (u + AHEAD < NSTEP) frags(u + AHEAD);
      if (u == NSTEP - AHEAD) {
#pragma unroll
        for (int q = 0; q < SK; ++q) {
          const int ks = wave + 4 * q;
          sa[q] = M::load(cb + sa_off + ks * M::KSTEP) * M::load(cb + sw_off + ks * M::KSTEP);
          sb[q] = M::load(cb + sb_off + ks * M::KSTEP);
        }
      }
      const frag fa0 = fk[u][0] * fx[u], fa1 = fk[u][1] * fx[u];
      acc00 = M::mma(fa0, fk[u][0], acc00);
      acc01 = M::mma(fa0, fk[u][1], acc01);
      acc11 = M::mma(fa1, fk[u][1], acc11);
#pragma unroll
      for (int it = u * NITEM / NSTEP; it < (u + 1) * NITEM / NSTEP; ++it) {
        store_item(Rs, nb, it);
        load_item(Rf, tn, it);
      }
    }
#pragma unroll
    for (int q = 0; q < SK; ++q) sacc = M::mma(sa[q], sb[q], sacc);
#if !defined(FM_HOSTSIM)
    __builtin_amdgcn_sched_barrier(0);
#endif
  };
  int nsnap = 0;
  auto tail = [&]() FM_ALWAYS_INLINE {
    const bool last = cur.t + TT >= cur.te;
    if (last) { finish_segment(nsnap); ++nsnap; }
    advance(cur);
    if (pf.valid) advance(pf);
  };
  while (true) {
    body(R1, R0, buf0, buf1);
    tail();
    if (!cur.valid) break;
    FM_SYNC();
    body(R0, R1, buf1, buf0);
    tail();
    if (!cur.valid) break;
    FM_SYNC();
  }
}
