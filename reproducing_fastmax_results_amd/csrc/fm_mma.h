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
  static FM_DEVICE frag load_perm(const fm_half* row, int s, int lh) {
    const fm_half4 lo = *reinterpret_cast<const fm_half4*>(row + 16 * s + 4 * lh);
    const fm_half4 hi = *reinterpret_cast<const fm_half4*>(row + 16 * s + 8 + 4 * lh);
    frag r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return r;
  }
  static FM_DEVICE frag from_acc(const fm_f32x16& c, int s) {
    frag r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = fm_half(c[8 * s + i]);
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
  static FM_DEVICE frag load_perm(const float* row, int s, int lh) { return row[8 * (s / 4) + 4 * lh + (s % 4)]; }
  static FM_DEVICE frag from_acc(const fm_f32x16& c, int s) { return c[s]; }
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
// Conversion to _Float16 saturates at the largest finite half so that an
// out-of-range input degrades instead of producing infinities.
template <typename E> struct CE;
template <> struct CE<fm_half> {
  static FM_DEVICE fm_half from(float x) {
    const float lim = 65504.f;
    x = x > lim ? lim : (x < -lim ? -lim : x);
    return fm_half(x);
  }
  // eight consecutive elements to LDS / workspace (16-byte aligned)
  static FM_DEVICE void st8(fm_half* p, const float in[8]) {
    fm_half8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = from(in[i]);
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
