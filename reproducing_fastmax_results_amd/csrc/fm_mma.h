// Matrix-core policies and element I/O helpers.
//
// Every contraction in this library is issued as a 32x32 MFMA tile on a 64-lane
// wavefront.  Lane l = 32*lh + lr supplies, for one k-step,
//     A[row = lr][k = lh*KPL .. lh*KPL+KPL-1]   and   B[k = same][col = lr],
// and owns the accumulator entries
//     D[row = 8*(e/4) + 4*lh + e%4][col = lr],   e = 0..15.
// Two instantiations: E = _Float16 (v_mfma_f32_32x32x16_f16, KPL = 8) for the
// bf16 interface and E = float (v_mfma_f32_32x32x2_f32, KPL = 1) for fp32.
// Because both operands use the same lane->k mapping, an accumulator can be fed
// back as the B operand of a following product as long as the A operand of that
// product is loaded with the accumulator's row order (`load_perm`).
#pragma once
#include "fm_platform.h"

template <typename E> struct Mma;

template <> struct Mma<fm_half> {
  typedef fm_half8 frag;
  static constexpr int KPL = 8;          // operand elements per lane per k-step
  static constexpr int KSTEP = 16;       // contraction length of one instruction
  static constexpr int ACC_KSTEPS = 2;   // k-steps that consume one 32-row accumulator
  static constexpr int PAD = 8;          // LDS row padding in elements (16 bytes)
  static constexpr int VEC = 8;          // elements per 16-byte chunk
  static FM_DEVICE fm_f32x16 mma(frag a, frag b, fm_f32x16 c) { return fm_mfma_f16(a, b, c); }
  static FM_DEVICE frag load(const fm_half* p) { return *reinterpret_cast<const fm_half8*>(p); }
  static FM_DEVICE frag splat(fm_half x) { frag r = {x, x, x, x, x, x, x, x}; return r; }
  static FM_DEVICE float elem(const frag& f, int i) { return float(f[i]); }   // operand element i of a lane's fragment
  // Transposed token tiles are stored with the 16 tokens of every group in the order
  // 0-3, 8-11, 4-7, 12-15 (`tperm`), so that the eight accumulator rows a lane needs for
  // accumulator k-step s (16s + 4lh + {0..3}, 16s + 8 + 4lh + {0..3}) are one 16-byte read.
  // A contraction over tokens does not care about their order as long as both operands
  // share it, so the same tiles serve the plain `load`.
  static FM_DEVICE int tperm(int t) { return (t & ~15) | (t & 3) | ((t & 8) >> 1) | ((t & 4) << 1); }
  static FM_DEVICE frag load_perm(const fm_half* row, int s, int lh) {
    return *reinterpret_cast<const fm_half8*>(row + 16 * s + 8 * lh);
  }
  static FM_DEVICE frag from_acc(const fm_f32x16& c, int s) {
    frag r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = fm_half(c[8 * s + i]);
    return r;
  }
  // The B fragment of k-step s of a row stored in natural order, in the k order a transposing read delivers its A
  // fragment (load_tr): elements 16 s + 4 lh + {0..3} and 16 s + 8 + 4 lh + {0..3}.
  static FM_DEVICE frag load_nat_perm(const fm_half* row, int s, int lh) {
    const fm_half4 lo = *reinterpret_cast<const fm_half4*>(row + 16 * s + 4 * lh);
    const fm_half4 hi = *reinterpret_cast<const fm_half4*>(row + 16 * s + 8 + 4 * lh);
    frag r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return r;
  }
  // The fragment load_perm would read from a transposed tile, taken from the ROW-MAJOR tile
  // instead (tokens x features, `pitch` elements per token) with two transposing reads: lane
  // (lr, lh) gets feature col0 + lr of the tokens tok0 + 4 lh + {0..3} and tok0 + 8 + 4 lh + {0..3},
  // the rows its accumulator k-step holds.  HAS_TR: the interface type for which this exists.
  static constexpr bool HAS_TR = true;
  static FM_DEVICE frag load_tr(const fm_half* tile, int pitch, int tok0, int col0, int lane) {
    const int lh = lane >> 5, half16 = (lane >> 4) & 1, s = (lane & 15) >> 2, q = lane & 3;
    const fm_half* p = tile + (tok0 + 4 * lh + s) * pitch + col0 + 16 * half16 + 4 * q;
    const fm_half4 lo = fm_lds_tr4(p), hi = fm_lds_tr4(p + 8 * pitch);
    frag r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return r;
  }
};

template <> struct Mma<float> {
  typedef float frag;
  static constexpr int KPL = 1;
  static constexpr int KSTEP = 2;
  static constexpr int ACC_KSTEPS = 16;
  static constexpr int PAD = 4;
  static constexpr int VEC = 4;
  static FM_DEVICE fm_f32x16 mma(frag a, frag b, fm_f32x16 c) { return fm_mfma_f32(a, b, c); }
  static FM_DEVICE frag load(const float* p) { return *p; }
  static FM_DEVICE frag splat(float x) { return x; }
  static FM_DEVICE float elem(const frag& f, int) { return f; }
  static FM_DEVICE int tperm(int t) { return t; }
  static FM_DEVICE frag load_perm(const float* row, int s, int lh) { return row[8 * (s / 4) + 4 * lh + (s % 4)]; }
  static constexpr bool HAS_TR = false;
  static FM_DEVICE frag load_tr(const float*, int, int, int, int) { return 0.f; }   // never called
  static FM_DEVICE frag from_acc(const fm_f32x16& c, int s) { return c[s]; }
  static FM_DEVICE frag load_nat_perm(const float*, int, int) { return 0.f; }   // never called
};

// Row index (0..31) of accumulator register e for a lane in half lh.
FM_DEVICE int fm_acc_row(int e, int lh) { return 8 * (e >> 2) + 4 * lh + (e & 3); }

FM_DEVICE fm_f32x16 fm_zero16() {
  fm_f32x16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}

// ---- interface element types (what the caller's tensors hold) -----------------
template <typename T> struct IO;
template <> struct IO<float> {
  static FM_DEVICE float ld(const float* p) { return *p; }
  static FM_DEVICE void st(float* p, float v) { *p = v; }
  // eight consecutive elements; `vec` says the address is 16-byte aligned
  static FM_DEVICE void ld8(const float* p, bool vec, float out[8]) {
    if (vec) {
      const fm_f32x4 a = *reinterpret_cast<const fm_f32x4*>(p);
      const fm_f32x4 b = *reinterpret_cast<const fm_f32x4*>(p + 4);
      out[0] = a[0]; out[1] = a[1]; out[2] = a[2]; out[3] = a[3];
      out[4] = b[0]; out[5] = b[1]; out[6] = b[2]; out[7] = b[3];
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) out[i] = p[i];
    }
  }
  static FM_DEVICE void st8(float* p, bool vec, const float in[8]) {
    if (vec) {
      fm_f32x4 a = {in[0], in[1], in[2], in[3]}, b = {in[4], in[5], in[6], in[7]};
      *reinterpret_cast<fm_f32x4*>(p) = a;
      *reinterpret_cast<fm_f32x4*>(p + 4) = b;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = in[i];
    }
  }
};
template <> struct IO<fm_bf16> {
  static FM_DEVICE float ld(const fm_bf16* p) { return fm_bf16_to_f32(*p); }
  static FM_DEVICE void st(fm_bf16* p, float v) { *p = fm_f32_to_bf16(v); }
  static FM_DEVICE void ld8(const fm_bf16* p, bool vec, float out[8]) {
    if (vec) {
      const fm_u32x4 u = *reinterpret_cast<const fm_u32x4*>(p);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t lo = u[i] << 16, hi = u[i] & 0xffff0000u;
        __builtin_memcpy(&out[2 * i], &lo, 4);
        __builtin_memcpy(&out[2 * i + 1], &hi, 4);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) out[i] = fm_bf16_to_f32(p[i]);
    }
  }
  static FM_DEVICE void st8(fm_bf16* p, bool vec, const float in[8]) {
    if (vec) {
      fm_u32x4 u;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        u[i] = uint32_t(fm_f32_to_bf16(in[2 * i])) | (uint32_t(fm_f32_to_bf16(in[2 * i + 1])) << 16);
      *reinterpret_cast<fm_u32x4*>(p) = u;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = fm_f32_to_bf16(in[i]);
    }
  }
};

// ---- compute element types ----------------------------------------------------
// Conversion to _Float16 rounds to nearest and does NOT saturate: a value beyond the largest finite
// half (65504) becomes an infinity, which every kernel carries through to a non-finite output.  An input
// outside the supported range therefore shows as inf / NaN in the results, never as a finite wrong number.
template <typename E> struct CE;
template <> struct CE<fm_half> {
  static FM_DEVICE fm_half from(float x) { return fm_half(x); }
  // eight consecutive elements to LDS / workspace (16-byte aligned)
  static FM_DEVICE void st8(fm_half* p, const float in[8]) {
    fm_half8 h;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      fm_f32x2 v = {in[i], in[i + 1]};
      const fm_half2 c = __builtin_convertvector(v, fm_half2);
      h[i] = c[0]; h[i + 1] = c[1];
    }
    *reinterpret_cast<fm_half8*>(p) = h;
  }
};
template <> struct CE<float> {
  static FM_DEVICE float from(float x) { return x; }
  static FM_DEVICE void st8(float* p, const float in[8]) {
    fm_f32x4 a = {in[0], in[1], in[2], in[3]}, b = {in[4], in[5], in[6], in[7]};
    *reinterpret_cast<fm_f32x4*>(p) = a;
    *reinterpret_cast<fm_f32x4*>(p + 4) = b;
  }
};

// ---- elementwise math on accumulator tiles --------------------------------------
// A tile is the 16 accumulator entries a lane owns (rows fm_acc_row(e, lh), one column).
// `edge` tiles apply the row window lo <= row <= hi (causal diagonal and sequence tail);
// interior tiles skip the test.  Results come back as B fragments (ACC_KSTEPS of them),
// ready for the next product.
//   fwd : P  = a0 + s (a1 + a2 s)                      and the lane's partial row-sum of P
//   dsc : dS = (a1 + 2 a2 s) (dp - c),  c one scalar per lane
//   dsr : the same with c per accumulator row (given as fragments in accumulator order)
//   both: P and dS (c per accumulator row) from one conversion of the score tile
// The _Float16 instantiation evaluates the polynomials on packed halves (v_pk_fma_f16)
// and sums with v_dot2_f32_f16, which keeps the vector pipe off the critical path.
template <typename E> struct TileMath;

template <> struct TileMath<float> {
  typedef float frag;
  struct Coef { float a0, a1, a2, ta2; };
  static FM_DEVICE Coef coef(float a0, float a1, float a2) { Coef c = {a0, a1, a2, 2.0f * a2}; return c; }
  static FM_DEVICE float fwd(const fm_f32x16& s, const Coef& k, bool edge, int lo, int hi, int lh, frag* pb) {
    float g = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float x = s[e];
      float pv = k.a0 + x * (k.a1 + k.a2 * x);
      if (edge) { const int r = fm_acc_row(e, lh); if (r < lo || r > hi) pv = 0.f; }
      g += pv;
      pb[e] = pv;
    }
    return g;
  }
  static FM_DEVICE void dsc(const fm_f32x16& s, const fm_f32x16& dp, float negc, const Coef& k, bool edge, int lo, int hi,
                            int lh, frag* db) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      float ds = (k.a1 + k.ta2 * s[e]) * (dp[e] + negc);
      if (edge) { const int r = fm_acc_row(e, lh); if (r < lo || r > hi) ds = 0.f; }
      db[e] = ds;
    }
  }
  static FM_DEVICE void dsr(const fm_f32x16& s, const fm_f32x16& dp, const float* negc, const Coef& k, bool edge, int lo,
                            int hi, int lh, frag* db) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      float ds = (k.a1 + k.ta2 * s[e]) * (dp[e] + negc[e]);
      if (edge) { const int r = fm_acc_row(e, lh); if (r < lo || r > hi) ds = 0.f; }
      db[e] = ds;
    }
  }
  static FM_DEVICE void both(const fm_f32x16& s, const fm_f32x16& dp, const float* negc, const Coef& k, bool edge, int lo,
                             int hi, int lh, frag* pb, frag* db) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float x = s[e];
      float pv = k.a0 + x * (k.a1 + k.a2 * x);
      float ds = (k.a1 + k.ta2 * x) * (dp[e] + negc[e]);
      if (edge) { const int r = fm_acc_row(e, lh); if (r < lo || r > hi) { pv = 0.f; ds = 0.f; } }
      pb[e] = pv;
      db[e] = ds;
    }
  }
};

// Completed-square forms (order 2, _Float16, dense tiles without states).  With a2 != 0,
//   f(s)  = a0 + a1 s + a2 s^2 = k1 * (h^2 + kc),   h = 2 a2 s + a1 = f'(s),   k1 = 1 / (4 a2),  kc = 4 a0 a2 - a1^2,
// so when the score product itself delivers h (own fragments multiplied by 2 a2, accumulator seeded with a1) the
// weight costs one packed multiply-add, W = h^2 + kc = f / k1, and the factor of the score gradient none; the
// constant k1 is taken out of the sums (o = F / g does not see it; g and dV are multiplied by it when stored).
// Likewise the accumulator of gh.v is seeded with -c, so dS = h * (gh.v - c) is one packed multiply.
//   wq   : W and the lane's partial row sum of W                        (forward)
//   dsq  : dS                                                           (dQ)
//   bothq: W and dS                                                     (dK and dV in one pass)
template <> struct TileMath<fm_half> {
  typedef fm_half8 frag;
  // every constant is one packed pair (one register); all arithmetic is written on pairs so
  // that it maps to v_cvt_pk_f16_f32 / v_pk_fma_f16 / v_pk_mul_f16 / v_pk_add_f16
  struct Coef { fm_half2 a0, a1, a2, ta2; };
  static FM_DEVICE fm_half2 pair(float x) { const fm_half h = CE<fm_half>::from(x); fm_half2 r = {h, h}; return r; }
  static FM_DEVICE Coef coef(float a0, float a1, float a2) {
    Coef c;
    c.a0 = pair(a0); c.a1 = pair(a1); c.a2 = pair(a2); c.ta2 = pair(2.0f * a2);
    return c;
  }
  static FM_DEVICE fm_half2 cvt2(float a, float b) {
    fm_f32x2 v = {a, b};
    return __builtin_convertvector(v, fm_half2);
  }
  static FM_DEVICE fm_half2 get2(const fm_half8& v, int i) {
    fm_half2 r = {v[2 * i], v[2 * i + 1]};
    return r;
  }
  static FM_DEVICE void put2(fm_half8& v, int i, fm_half2 x) { v[2 * i] = x[0]; v[2 * i + 1] = x[1]; }
  // zero the entries of both fragments whose accumulator row is outside [lo, hi]
  static FM_DEVICE void window_frags(frag* f, int lo, int hi, int lh) {
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int r = fm_acc_row(8 * ss + i, lh);
        if (r < lo || r > hi) f[ss][i] = fm_half(0.f);
      }
  }
  static FM_DEVICE float fwd(const fm_f32x16& s, const Coef& k, bool edge, int lo, int hi, int lh, frag* pb) {
    const fm_half2 one = {fm_half(1.f), fm_half(1.f)};
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = 8 * ss + 2 * i;
        const fm_half2 x = cvt2(s[e], s[e + 1]);
        put2(pb[ss], i, (x * k.a2 + k.a1) * x + k.a0);
      }
    if (edge) { FM_KEEP_BRANCH(); window_frags(pb, lo, hi, lh); }
    float g = 0.f;
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) g = fm_dot2(get2(pb[ss], i), one, g);
    return g;
  }
  // Own = queries (dsc): c of the lane's query is subtracted as a half from the rounded gh.v (its rounding moves the
  // query's own gradient by a few parts in a thousand at worst).  Own = keys (dsr, both): c is taken off gh.v in
  // fp32, before the difference is rounded: the two are of one size, and an error in c has one sign along a query's
  // whole row of keys, so over the keys it adds up in sum_j dk_j (what a projection's weight gradient sees) instead
  // of averaging out.
  static FM_DEVICE void dsc(const fm_f32x16& s, const fm_f32x16& dp, float negc, const Coef& k, bool edge, int lo, int hi,
                            int lh, frag* db) {
    const fm_half2 nc = pair(negc);
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = 8 * ss + 2 * i;
        const fm_half2 x = cvt2(s[e], s[e + 1]);
        put2(db[ss], i, (x * k.ta2 + k.a1) * (cvt2(dp[e], dp[e + 1]) + nc));
      }
    if (edge) { FM_KEEP_BRANCH(); window_frags(db, lo, hi, lh); }
  }
  static FM_DEVICE void dsr(const fm_f32x16& s, const fm_f32x16& dp, const float* negc, const Coef& k, bool edge, int lo,
                            int hi, int lh, frag* db) {
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = 8 * ss + 2 * i;
        const fm_half2 x = cvt2(s[e], s[e + 1]);
        put2(db[ss], i, (x * k.ta2 + k.a1) * cvt2(dp[e] + negc[e], dp[e + 1] + negc[e + 1]));
      }
    if (edge) { FM_KEEP_BRANCH(); window_frags(db, lo, hi, lh); }
  }
  static FM_DEVICE void both(const fm_f32x16& s, const fm_f32x16& dp, const float* negc, const Coef& k, bool edge, int lo,
                             int hi, int lh, frag* pb, frag* db) {
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = 8 * ss + 2 * i;
        const fm_half2 x = cvt2(s[e], s[e + 1]);
        put2(pb[ss], i, (x * k.a2 + k.a1) * x + k.a0);
        put2(db[ss], i, (x * k.ta2 + k.a1) * cvt2(dp[e] + negc[e], dp[e + 1] + negc[e + 1]));
      }
    if (edge) { FM_KEEP_BRANCH(); window_frags(pb, lo, hi, lh); window_frags(db, lo, hi, lh); }
  }
  static FM_DEVICE float wq(const fm_f32x16& h, fm_half2 kc, bool edge, int lo, int hi, int lh, frag* pb) {
    const fm_half2 one = {fm_half(1.f), fm_half(1.f)};
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = 8 * ss + 2 * i;
        const fm_half2 x = cvt2(h[e], h[e + 1]);
        put2(pb[ss], i, x * x + kc);
      }
    if (edge) { FM_KEEP_BRANCH(); window_frags(pb, lo, hi, lh); }
    float g = 0.f;
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) g = fm_dot2(get2(pb[ss], i), one, g);
    return g;
  }
  static FM_DEVICE void dsq(const fm_f32x16& h, const fm_f32x16& dpc, bool edge, int lo, int hi, int lh, frag* db) {
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = 8 * ss + 2 * i;
        put2(db[ss], i, cvt2(h[e], h[e + 1]) * cvt2(dpc[e], dpc[e + 1]));
      }
    if (edge) { FM_KEEP_BRANCH(); window_frags(db, lo, hi, lh); }
  }
  static FM_DEVICE void bothq(const fm_f32x16& h, const fm_f32x16& dpc, fm_half2 kc, bool edge, int lo, int hi, int lh,
                              frag* pb, frag* db) {
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = 8 * ss + 2 * i;
        const fm_half2 x = cvt2(h[e], h[e + 1]);
        put2(pb[ss], i, x * x + kc);
        put2(db[ss], i, x * cvt2(dpc[e], dpc[e + 1]));
      }
    if (edge) { FM_KEEP_BRANCH(); window_frags(pb, lo, hi, lh); window_frags(db, lo, hi, lh); }
  }
};

// The 16 accumulator entries of a lane, all equal to x, as a value the optimiser cannot take apart: kept in
// registers across a loop and handed to the first matrix instruction of every tile as its addend (a seed the
// compiler could see through would be rebuilt with 16 moves per tile).
FM_DEVICE fm_f32x16 fm_seed16(float x) {
  fm_f32x16 r;
#pragma unroll
  for (int i = 0; i < 16; ++i) r[i] = x;
#if !defined(FM_HOSTSIM)
  asm volatile("" : "+v"(r));
#endif
  return r;
}
