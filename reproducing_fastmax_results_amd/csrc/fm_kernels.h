// Fastmax kernels for gfx950 (also compiled by the host simulator for tests).
//
// Math (per batch*head), s_ij = q_i.k_j / tau, f(s) = a0 + a1 s + a2 s^2:
//     F_i = sum_j M_ij f(s_ij) v_j,  g_i = sum_j M_ij f(s_ij),  o_i = F_i / g_i.
// The sequence is cut into segments of L tokens.  Keys of earlier segments (all
// keys when there is no mask) reach a query through moment states
//     T[a][r][c] = coef * sum_t x_ta p_tr r_tc     (a < D: order 2,  a = D: order 1, x = 1)
// and keys of the query's own segment through dense masked tiles f(Q K^T).
// Reference behaviour being reproduced: fastmax_cuda_forward.cu:23-280 (running
// sums per thread) and fastattention_einops.py:186-322 (cumsum of outer products).
//
// All contractions are computed "transposed": the accumulator column (lane) is
// the token, the accumulator rows are features.  That keeps one token per lane,
// so a per-token scalar (q_ia, 1/g_i, c_i) is a per-lane scalar.
#pragma once
#include "fastmax_hip.h"
#include "fm_mma.h"

#if defined(FM_HOSTSIM)
#define FM_SHARED static
#else
#define FM_SHARED __shared__
#endif

static constexpr int FM_THREADS = 256;   // four wavefronts per workgroup, everywhere

// Workgroups are handed to the 8 XCDs round-robin in launch order, and each XCD has its own
// L2.  All workgroups of one batch*head read the same tiles and states, so the launch index
// is remapped to put them on one XCD: with `units` workgroups per batch*head and nbh a
// multiple of 8, launch index id runs on XCD id % 8 and becomes unit (id / 8) % units of
// batch*head id % 8 + 8 * ((id / 8) / units).  Otherwise the plain 2-D index is used.
FM_DEVICE void fm_xcd_map(int units, int nbh, int& unit, int& bh) {
  const int id = FM_BID_X + FM_GDIM_X * FM_BID_Y;
  if ((nbh & 7) == 0) {
    const int x = id & 7, j = id >> 3;
    unit = j % units;
    bh = x + 8 * (j / units);
  } else {
    unit = id % units;
    bh = id / units;
  }
}

// ------------------------------------------------------------------------------
// tile movers (global -> registers -> LDS), 16-byte chunks, 256 threads
// ------------------------------------------------------------------------------
template <typename E, int ROWS, int TT>
struct TileRegs {
  static constexpr int VEC = Mma<E>::VEC;
  static constexpr int CPR = TT / VEC;                 // chunks per row
  static constexpr int TOTAL = ROWS * CPR;
  static constexpr int N = (TOTAL + FM_THREADS - 1) / FM_THREADS;
  fm_u32x4 r[N];
  // src points at (row 0, first token of the tile); rows are row_stride apart
  // (src is the same in every lane; the per-lane part is an unsigned 32-bit element offset, so
  // the address is a scalar base plus a vector offset and no 64-bit pointer is kept per lane)
  FM_DEVICE void load(const E* src, int row_stride, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int c = tid + FM_THREADS * i;
      if (TOTAL % FM_THREADS == 0 || c < TOTAL) {
        const uint32_t row = uint32_t(c / CPR), col = uint32_t((c % CPR) * VEC);
        const uint32_t off = row * uint32_t(row_stride) + col;
        r[i] = *reinterpret_cast<const fm_u32x4*>(src + off);
      }
    }
  }
  FM_DEVICE void store(E* lds, int pitch, int tid) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int c = tid + FM_THREADS * i;
      if (TOTAL % FM_THREADS == 0 || c < TOTAL) {
        const int row = c / CPR, col = (c % CPR) * VEC;
        *reinterpret_cast<fm_u32x4*>(lds + row * pitch + col) = r[i];
      }
    }
  }
  // one chunk of the thread at a time (tiles of a whole number of chunks per thread)
  FM_DEVICE void load_part(const E* src, int row_stride, int tid, int i) {
    static_assert(TOTAL % FM_THREADS == 0 || TOTAL <= FM_THREADS, "whole chunks per thread");
    const int c = TOTAL <= FM_THREADS ? tid % TOTAL : tid + FM_THREADS * i;
    r[i] = *reinterpret_cast<const fm_u32x4*>(src + uint32_t(c / CPR) * uint32_t(row_stride) + uint32_t((c % CPR) * VEC));
  }
  FM_DEVICE void store_part(E* lds, int pitch, int tid, int i) const {
    const int c = TOTAL <= FM_THREADS ? tid % TOTAL : tid + FM_THREADS * i;
    *reinterpret_cast<fm_u32x4*>(lds + (c / CPR) * pitch + (c % CPR) * VEC) = r[i];
  }
  // The same without a branch, for a tile of fewer chunks than threads: the surplus threads repeat the work of the
  // first ones (same addresses, same data), so the instructions can be scheduled among others.
  FM_DEVICE void load_wrapped(const E* src, int row_stride, int tid) {
    static_assert(N == 1 && TOTAL <= FM_THREADS, "a tile of at most one chunk per thread");
    const int c = tid % TOTAL;
    r[0] = *reinterpret_cast<const fm_u32x4*>(src + uint32_t(c / CPR) * uint32_t(row_stride) + uint32_t((c % CPR) * VEC));
  }
  FM_DEVICE void store_wrapped(E* lds, int pitch, int tid) const {
    static_assert(N == 1 && TOTAL <= FM_THREADS, "a tile of at most one chunk per thread");
    const int c = tid % TOTAL;
    *reinterpret_cast<fm_u32x4*>(lds + (c / CPR) * pitch + (c % CPR) * VEC) = r[0];
  }
};

// Rows of a caller tensor (interface type, strided, bounds-checked) -> LDS in the
// compute type.  ROWS x DH elements, eight elements per chunk.
template <typename TIO, typename E, int ROWS, int DH>
struct RowRegs {
  static constexpr int CPR = DH / 8;
  static constexpr int TOTAL = ROWS * CPR;
  static constexpr int N = (TOTAL + FM_THREADS - 1) / FM_THREADS;
  float v[N][8];
  // base points at (token 0, feature 0) of this batch*head; rows row0..row0+ROWS-1
  FM_DEVICE void load(const TIO* base, int64_t s_n, bool vec, int row0, int nrows, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int c = tid + FM_THREADS * i;
      if (TOTAL % FM_THREADS == 0 || c < TOTAL) {
        const int row = row0 + c / CPR, col = (c % CPR) * 8;
        if (row < nrows) {
          IO<TIO>::ld8(base + int64_t(row) * s_n + col, vec, v[i]);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) v[i][j] = 0.f;
        }
      }
    }
  }
  FM_DEVICE void store(E* lds, int pitch, int tid, float scale) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int c = tid + FM_THREADS * i;
      if (TOTAL % FM_THREADS == 0 || c < TOTAL) {
        const int row = c / CPR, col = (c % CPR) * 8;
        float w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = v[i][j] * scale;
        CE<E>::st8(lds + row * pitch + col, w);
      }
    }
  }
};

// A caller tensor: base pointer, strides in elements, whether 16-byte accesses are aligned.
template <typename TIO> struct TRef {
  TIO* p; int64_t s_bh, s_n; int vec; int64_t s_b; int heads;
  // first element of batch*head slice bh (one stride, or batch and head strides when heads > 1)
  FM_DEVICE TIO* base(int bh) const {
    return heads > 1 ? p + int64_t(bh / heads) * s_b + int64_t(bh % heads) * s_bh : p + int64_t(bh) * s_bh;
  }
};

// host side: TRef of a caller pointer and its FastmaxStrides
template <typename T> inline bool fm_vec_ok(const void* ptr, const FastmaxStrides& s) {
  const int64_t a = 16 / int64_t(sizeof(T));          // elements per 16 bytes
  return (reinterpret_cast<uintptr_t>(ptr) % 16 == 0) && (s.n % a == 0) && (s.bh % a == 0) &&
         (s.heads <= 1 || s.b % a == 0);
}
template <typename T> inline TRef<T> fm_ref(T* ptr, const FastmaxStrides& s) {
  TRef<T> r;
  r.p = ptr; r.s_bh = s.bh; r.s_n = s.n; r.vec = fm_vec_ok<T>(ptr, s) ? 1 : 0;
  r.s_b = s.heads > 1 ? s.b : 0; r.heads = s.heads > 1 ? s.heads : 0;
  return r;
}

// ------------------------------------------------------------------------------
// Max-norm normalisation folded into the loads:  x_hat = lim * x / max_n ||x_n||_2  per batch*head
// (transformer/model.py:97-102; apply_norm of fastmax_cuda_forward.cu:326-338 makes this a pass of its own
// that reads and rewrites the tensor).  One statistics pass (k_maxnorm_keys in fm_norm.h) leaves one 64-bit
// key per 256 tokens: the bits of the largest squared token norm in the high half and ~token in the low
// half, so that an integer maximum finds the largest norm and, among equal ones, the first token.  Every
// kernel that loads such a tensor joins the keys of its batch*head (the same values in the same order
// everywhere, so all agree on the bits) and multiplies by lim / max-norm as it converts the rows.
// ------------------------------------------------------------------------------
struct NormFold {
  const unsigned long long* keys;   // [bh][nblk], or null: the tensor is taken as it is
  int nblk;
  float lim;
};
static constexpr int FM_MAXNORM_TOKENS = 256;
inline int fm_maxnorm_blocks(int n) { return (n + FM_MAXNORM_TOKENS - 1) / FM_MAXNORM_TOKENS; }
// A slice whose largest squared norm is not above this value (all zeros: padding) is mapped to zeros.
static constexpr float FM_MAXNORM_FLOOR = 1e-30f;

FM_DEVICE unsigned long long fm_shfl_xor_u64(unsigned long long v, int m) {
  const int lo = fm_shfl_xor_i(int(uint32_t(v)), m), hi = fm_shfl_xor_i(int(uint32_t(v >> 32)), m);
  return (static_cast<unsigned long long>(uint32_t(hi)) << 32) | uint32_t(lo);
}
// largest squared norm m2 and its token of one batch*head; every lane of the wavefront must call it
FM_DEVICE void fm_maxnorm_join(const unsigned long long* keys, int nblk, int lane, float& m2, int& nstar) {
  unsigned long long k = 0;
  constexpr int UB = 4;                                  // loads in flight per round (see fm_grad_scale)
  for (int i0 = lane; i0 < nblk; i0 += 64 * UB) {
    unsigned long long x[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u) x[u] = (i0 + 64 * u < nblk) ? keys[i0 + 64 * u] : 0ull;
#pragma unroll
    for (int u = 0; u < UB; ++u) k = x[u] > k ? x[u] : k;
  }
#pragma unroll
  for (int w = 1; w < 64; w <<= 1) { const unsigned long long o = fm_shfl_xor_u64(k, w); k = o > k ? o : k; }
  const uint32_t bits = uint32_t(k >> 32);
  __builtin_memcpy(&m2, &bits, 4);
  nstar = int(~uint32_t(k));
}
// lim / max-norm of batch*head bh (1 when the fold is off, 0 for an all-zero slice)
FM_DEVICE float fm_norm_factor(const NormFold& f, int bh, int lane) {
  if (!f.keys) return 1.0f;
  float m2; int nstar;
  fm_maxnorm_join(f.keys + int64_t(bh) * f.nblk, f.nblk, lane, m2, nstar);
  return m2 > FM_MAXNORM_FLOOR ? f.lim * fm_rsqrtf(m2) : 0.0f;
}

// ------------------------------------------------------------------------------
// k_transpose: x (bh, n, DH) strided, interface type  ->  compute type, multiplied by
// `scale`, zero for tokens >= n:  xt [bh][DH][npad] (transposed) and, when xr is not
// null, xr [bh][npad][DH] (row-major); xt may be null as well (the _Float16 token kernels read
// transposed fragments out of row tiles; only the state walk needs xt).  The token-side kernels stage their tiles from
// these copies with plain 16-byte moves.  Two tensors of the same length (k and v) go in one
// launch: grid (npad/64, bh, 2), the second set of arguments serves z = 1.
// ------------------------------------------------------------------------------
template <typename TIO, typename E> struct TransposeJob { TRef<const TIO> x; E* xt; E* xr; float scale; NormFold fold; };

template <typename TIO, typename E, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS)
k_transpose(TransposeJob<TIO, E> j0, TransposeJob<TIO, E> j1, int n, int npad) {
  constexpr int PT = 64 + Mma<E>::PAD;
  constexpr int VEC = Mma<E>::VEC;
  FM_SHARED E tile[DH * PT];
  const int tid = FM_TID_X, t0 = FM_BID_X * 64, bh = FM_BID_Y;
  const bool second = FM_BID_Z != 0;
  const TRef<const TIO> x = second ? j1.x : j0.x;
  E* FM_RESTRICT xt = second ? j1.xt : j0.xt;
  E* FM_RESTRICT xr = second ? j1.xr : j0.xr;
  const float scale = (second ? j1.scale : j0.scale) * fm_norm_factor(second ? j1.fold : j0.fold, bh, tid & 63);
  const TIO* xb = x.base(bh);
  const int64_t s_n = x.s_n;
  const int vec = x.vec;
  for (int c = tid; c < 64 * (DH / 8); c += FM_THREADS) {
    const int tok = c / (DH / 8), d0 = (c % (DH / 8)) * 8;
    float v[8];
    if (t0 + tok < n) {
      IO<TIO>::ld8(xb + int64_t(t0 + tok) * s_n + d0, vec != 0, v);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] *= scale;
    if (xr) CE<E>::st8(xr + (int64_t(bh) * npad + t0 + tok) * DH + d0, v);
    if (xt) {
#pragma unroll
      for (int j = 0; j < 8; ++j) tile[(d0 + j) * PT + Mma<E>::tperm(tok)] = CE<E>::from(v[j]);
    }
  }
  if (!xt) return;                                     // only the row-major copy was asked for
  FM_SYNC();
  E* ob = xt + int64_t(bh) * DH * npad + t0;
  for (int c = tid; c < DH * (64 / VEC); c += FM_THREADS) {
    const int d = c / (64 / VEC), tk = (c % (64 / VEC)) * VEC;
    *reinterpret_cast<fm_u32x4*>(ob + int64_t(d) * npad + tk) =
        *reinterpret_cast<const fm_u32x4*>(&tile[d * PT + tk]);
  }
}

// ------------------------------------------------------------------------------
// Scale of the upstream gradient.  Every gradient is linear in gh_i = dO_i / g_i, and the size of dO is the
// caller's: a loss averaged over tens of thousands of tokens hands over dO of 1e-6 and less, and g grows with
// the token index, so gh can lie anywhere - far below what _Float16 holds included.  k_grad_scale finds, per
// workgroup of 64 tokens, the largest |dO_if| / |g_i|; every later kernel joins the partial maxima of its
// batch*head (fm_grad_scale: the same few values in the same order everywhere, so all kernels agree on the
// bits) into the power of two that brings the largest |gh| element of the batch*head to [32, 64), multiplies
// gh by it when it is formed and divides the gradients by it when they are stored.  Inside a batch*head gh
// varies by about the sequence length (g_i ~ i), which leaves the smallest rows of a 65536-token sequence near
// 1e-3, well inside the normal _Float16 range, and the dot products gh.v and gh.o (64 terms) below 65504.
// grid (ceil(n / 64), bh); part [bh][nblk].
// ------------------------------------------------------------------------------
static constexpr int FM_GS_TOKENS = 64;
inline int fm_grad_scale_blocks(int n) { return (n + FM_GS_TOKENS - 1) / FM_GS_TOKENS; }

template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS) k_grad_scale(TRef<const TIO> d_o, TRef<const float> g, int n, float* FM_RESTRICT part) {
  constexpr int EPT = DH / 4, NP = FM_GS_TOKENS / 64;
  FM_SHARED float wmax[4];
  const int tid = FM_TID_X, bh = FM_BID_Y;
  const int tok0 = FM_BID_X * FM_GS_TOKENS + (tid >> 2), d0 = (tid & 3) * EPT;
  float v[NP][EPT], gi[NP];
  // all loads first; rows past the end re-read the last row (every lane takes part in the shuffles)
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int tok = tok0 + 64 * p, tk = tok < n ? tok : n - 1;
    gi[p] = g.base(bh)[int64_t(tk) * g.s_n];
#pragma unroll
    for (int j = 0; j < EPT; j += 8) IO<TIO>::ld8(d_o.base(bh) + int64_t(tk) * d_o.s_n + d0 + j, d_o.vec != 0, &v[p][j]);
  }
  float mx = 0.f;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < EPT; ++j) m = fm_fmaxf(m, v[p][j] < 0.f ? -v[p][j] : v[p][j]);
    const float ga = gi[p] < 0.f ? -gi[p] : gi[p];
    mx = fm_fmaxf(mx, m / ga);                       // fmax drops a NaN (0 / 0); an infinity (g = 0) is kept and ignored by the consumers
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) mx = fm_fmaxf(mx, fm_shfl_xor(mx, m));
  if ((tid & 63) == 0) wmax[tid >> 6] = mx;
  FM_SYNC();
  if (tid == 0) part[int64_t(bh) * FM_GDIM_X + FM_BID_X] = fm_fmaxf(fm_fmaxf(wmax[0], wmax[1]), fm_fmaxf(wmax[2], wmax[3]));
}

// The power of two described above, from the nblk partial maxima of one batch*head; 1 when there are none
// (part == null: the fp32 kernels need no scaling) or when the maximum is zero or not finite.  Every lane of the
// wavefront must call it; every lane gets the same value.
FM_DEVICE float fm_grad_scale(const float* part, int nblk, int lane) {
  if (!part) return 1.0f;
  float m = 0.f;
  // sixteen loads in flight per round: a long sequence has a thousand parts, and one load per round trip would
  // make this a chain of memory latencies at the start of every workgroup
  constexpr int UB = 16;
  for (int i0 = lane; i0 < nblk; i0 += 64 * UB) {
    float x[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u) x[u] = (i0 + 64 * u < nblk) ? part[i0 + 64 * u] : 0.f;
#pragma unroll
    for (int u = 0; u < UB; ++u) if (x[u] < 3.0e38f) m = fm_fmaxf(m, x[u]);
  }
#pragma unroll
  for (int w = 1; w < 64; w <<= 1) m = fm_fmaxf(m, fm_shfl_xor(m, w));
  if (!(m > 0.f)) return 1.0f;
  uint32_t bits;
  __builtin_memcpy(&bits, &m, 4);
  int eb = int((bits >> 23) & 0xffu);                 // m = 1.x * 2^(eb - 127)  (eb = 0: subnormal, treated as 2^-126)
  if (eb < 1) eb = 1;
  int sb = 259 - eb;                                  // 2^(5 - (eb - 127))
  if (sb > 254) sb = 254;
  if (sb < 1) sb = 1;
  const uint32_t out = uint32_t(sb) << 23;
  float r;
  __builtin_memcpy(&r, &out, 4);
  return r;
}

// ------------------------------------------------------------------------------
// k_prep_bwd: per token  gh = gscale * dO / g,  c = gh . o,  q' = qscale * q ; writes
//   gh  [bh][npad][DH]  (row-major, compute type)      ght [bh][DH][npad]
//   qt  [bh][DH][npad]  (q' transposed)                 qct [bh][DH][npad]  (c_i q'_i; skipped when null:
//                                                        only the state walk reads it)
//   qr  [bh][npad][DH]  (q' row-major)
//   cv  [bh][npad]      (c, fp32)
// gscale is the power of two of fm_grad_scale (see k_grad_scale): it keeps gh inside the _Float16
// range; every gradient is linear in (gh, c) and is divided by gscale again when it is stored.
// Tokens >= n are written as zeros.  grid (npad/64, bh).
// Reference: div_grad_output, fastmax_cuda_backward.cu:494-501, and the
// "grad * o" row sums of fastattention_einops.py:405-407.
// ------------------------------------------------------------------------------
template <typename TIO, typename E, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS)
k_prep_bwd(TRef<const TIO> q, TRef<const TIO> o, TRef<const TIO> d_o, TRef<const float> g, int n, int npad, E* FM_RESTRICT gh, E* FM_RESTRICT ght,
           E* FM_RESTRICT qt, E* FM_RESTRICT qct, E* FM_RESTRICT qr, float* FM_RESTRICT cv, float qscale0,
           const float* FM_RESTRICT gpart, int gnblk, NormFold qfold, const fm_half* FM_RESTRICT ores) {
  // ores: what bf16 rounding took away from o ([bh][npad][DH] halves, written by a forward that kept its workspace), or null
  constexpr int PT = 64 + Mma<E>::PAD;
  constexpr int VEC = Mma<E>::VEC;
  constexpr int EPT = DH / 4;                      // elements per thread (4 threads per token)
  FM_SHARED E tg[DH * PT];
  FM_SHARED E tq[DH * PT];
  FM_SHARED E tc[DH * PT];
  const int tid = FM_TID_X, t0 = FM_BID_X * 64, bh = FM_BID_Y;
  const int tok = tid >> 2, part = tid & 3, d0 = part * EPT;
  const int row = t0 + tok;
  const float gscale = fm_grad_scale(gpart ? gpart + int64_t(bh) * gnblk : nullptr, gnblk, tid & 63);
  const float qscale = qscale0 * fm_norm_factor(qfold, bh, tid & 63);
  float vg[EPT], vq[EPT];
  float csum = 0.f;
  if (row < n) {
    // every load of the thread is issued before the first result is used
    float a[EPT], b[EPT], c[EPT];
    fm_half8 r[EPT / 8];
    const float gi = g.base(bh)[int64_t(row) * g.s_n];
#pragma unroll
    for (int j = 0; j < EPT; j += 8) {
      IO<TIO>::ld8(d_o.base(bh) + int64_t(row) * d_o.s_n + d0 + j, d_o.vec != 0, &a[j]);
      IO<TIO>::ld8(o.base(bh) + int64_t(row) * o.s_n + d0 + j, o.vec != 0, &b[j]);
      IO<TIO>::ld8(q.base(bh) + int64_t(row) * q.s_n + d0 + j, q.vec != 0, &c[j]);
      r[j / 8] = ores ? *reinterpret_cast<const fm_half8*>(ores + (int64_t(bh) * npad + row) * DH + d0 + j)
                      : Mma<fm_half>::splat(fm_half(0.f));
    }
    const float ginv = gscale / gi;
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      vg[j] = a[j] * ginv;
      csum += vg[j] * (b[j] + float(r[j / 8][j % 8]));
      vq[j] = c[j] * qscale;
    }
  } else {
#pragma unroll
    for (int j = 0; j < EPT; ++j) { vg[j] = 0.f; vq[j] = 0.f; }
  }
  csum += fm_shfl_xor(csum, 1);
  csum += fm_shfl_xor(csum, 2);
  if (part == 0) cv[int64_t(bh) * npad + t0 + Mma<E>::tperm(tok)] = csum;
  E* ghrow = gh + (int64_t(bh) * npad + row) * DH + d0;
  E* qrrow = qr + (int64_t(bh) * npad + row) * DH + d0;
#pragma unroll
  for (int j = 0; j < EPT; j += 8) { CE<E>::st8(ghrow + j, &vg[j]); CE<E>::st8(qrrow + j, &vq[j]); }
  if (!qt) return;                                     // ght, qt, qct: only the state walk and the fp32 kernels read them
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    tg[(d0 + j) * PT + Mma<E>::tperm(tok)] = CE<E>::from(vg[j]);
    tq[(d0 + j) * PT + Mma<E>::tperm(tok)] = CE<E>::from(vq[j]);
    tc[(d0 + j) * PT + Mma<E>::tperm(tok)] = CE<E>::from(vq[j] * csum);
  }
  FM_SYNC();
  const int64_t ob = int64_t(bh) * DH * npad + t0;
  for (int c = tid; c < DH * (64 / VEC); c += FM_THREADS) {
    const int d = c / (64 / VEC), tk = (c % (64 / VEC)) * VEC;
    const int64_t off = ob + int64_t(d) * npad + tk;
    *reinterpret_cast<fm_u32x4*>(ght + off) = *reinterpret_cast<const fm_u32x4*>(&tg[d * PT + tk]);
    *reinterpret_cast<fm_u32x4*>(qt + off) = *reinterpret_cast<const fm_u32x4*>(&tq[d * PT + tk]);
    if (qct) *reinterpret_cast<fm_u32x4*>(qct + off) = *reinterpret_cast<const fm_u32x4*>(&tc[d * PT + tk]);
  }
}

// ------------------------------------------------------------------------------
// Moment states.
//   big   [slot][a = 0..DH][r][c]   compute type;  a < DH: coef2 * sum x_a p_r r_c,
//                                                  a = DH: coef1 * sum p_r r_c
//   small [slot]{ Z[DH][DH], va[DH], vb[DH] } fp32;  Z = coefz * sum za_r zb_c,
//                                   va = coefva * sum za,  vb = coefvb * sum p (or sum r)
//   big2  [slot][a][c][r] = coefb * (same sums): the transposed tiles.  The state of
//         (x, p, r) read with (r, p) exchanged is the state of (x, r, p), so one walk
//         serves two consumers (dK wants [a][m][c], dV wants [a][c][m]).
// ------------------------------------------------------------------------------
// `big` is padded to DH + 4 values of a so that a reader may fetch whole slabs of
// up to four values of a starting at any a <= DH without leaving the state.
template <int DH> struct StateDims {
  static constexpr int64_t BIG = int64_t(DH + 4) * DH * DH;
  static constexpr int64_t SMALL = int64_t(DH) * DH + 2 * DH;
  static constexpr int64_t SLAB = int64_t(DH) * DH;
  static constexpr int PAD_SLABS = 3;                  // readers fetch up to four slabs at a time
  // Elements between the slots of two consecutive segments in a `big` array, and where the order-1
  // slab lies inside a slot.  With order-2 states a slot is the D slabs T[a], the order-1 slab and
  // the padding; without them it is the order-1 slab alone (the padding follows the last slot), so
  // that the hundreds of small states of a long order-1 sequence lie side by side instead of half
  // a megabyte apart.
  static FM_HOST_DEVICE int64_t stride(bool quad) { return quad ? BIG : SLAB; }
  static FM_HOST_DEVICE int64_t slab1(bool quad) { return quad ? DH * SLAB : 0; }
};

enum { FM_WALK_PREFIX = 0, FM_WALK_SUFFIX = 1, FM_WALK_TOTAL = 2 };

enum { FM_SRC_P = 0, FM_SRC_R = 1, FM_SRC_Z = 2 };

template <typename E> struct BuildArgs {
  const E* xt; const E* pt; const E* rt;   // [bh][DH][npad] transposed operands
  const E* zt;                             // optional third operand (rows of the Z product), or null
  int za_sel, zb_sel;                      // Z = sum za_r zb_c with za, zb chosen among p, r, zt
  int npad, nseg, L, mode, quad;
  E* big; float* small;                    // [bh][nslots] states
  E* big2;                                 // optional second copy with every [r][c] tile transposed
  int nslots;
  int vb_from_r;                           // vb sums the r operand instead of p
  float coef2, coef1, coefz, coefva, coefvb;
  float coef2b, coef1b;                    // coefficients of the transposed copy
  int skip_big;                            // order 2: the snapshot goes to big2 only (nobody reads the first layout); the
                                           // order-1 tile and the lower-order sums are written as always
  int seg_parallel;                        // grid z = walk step: every workgroup sums one segment only and
                                           // k_state_scan turns the per-segment sums into prefix / suffix states
  // Order-1 sums from row-major operands (k_build1_rows; null: the transposed operands above are read):
  const E* pr; const E* rr;                // [bh][npad][DH] rows of the p and r operands
  const float* cw;                         // [bh][npad] per-token weights, fp32 (stored in `tperm` order): the third
                                           // operand is then cw_t * p_t, and zt is not read; or null
};

FM_DEVICE void fm_walk_step(int mode, int nseg, int L, int npad, int w, int& tb, int& te, int& slot) {
  if (mode == FM_WALK_PREFIX) { tb = w * L; te = tb + L; slot = w + 1; }
  else if (mode == FM_WALK_SUFFIX) {
    const int s = nseg - 1 - w;
    tb = s * L; te = tb + L; if (te > npad) te = npad; slot = s - 1;
  } else { tb = 0; te = npad; slot = 0; }
}

// One reduced lower-order 32x32 tile (v: the lane's 16 accumulator values) to its place in the
// state of `slot`: tl < NT*NT the order-1 tile (and its transposed copy), then the Z tiles, then
// the two vector sums (column 0 of their tiles).
template <typename E, int DH>
FM_DEVICE void fm_put_small(const BuildArgs<E>& A, E* big, E* big2, float* ds, int slot, int tl, const float* v, int lr,
                            int lh) {
  constexpr int NT = DH / 32;
  if (tl < NT * NT) {
    const int r0 = 32 * (tl / NT), c = 32 * (tl % NT) + lr;
    E* d1 = big + int64_t(slot) * StateDims<DH>::stride(A.quad != 0) + StateDims<DH>::slab1(A.quad != 0);
#pragma unroll
    for (int e = 0; e < 16; ++e) d1[(r0 + fm_acc_row(e, lh)) * DH + c] = CE<E>::from(A.coef1 * v[e]);
    if (big2) {
      E* d2 = big2 + int64_t(slot) * StateDims<DH>::stride(A.quad != 0) + StateDims<DH>::slab1(A.quad != 0);
      // a lane owns four consecutive rows four times over: one 8-byte (16-byte for float) store each
      struct alignas(4 * sizeof(E)) Four { E v[4]; };
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        Four f;
#pragma unroll
        for (int u = 0; u < 4; ++u) f.v[u] = CE<E>::from(A.coef1b * v[4 * g + u]);
        *reinterpret_cast<Four*>(d2 + c * DH + r0 + fm_acc_row(4 * g, lh)) = f;
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

// k_build (order 2): one workgroup per (group of 4*NA values of a, batch*head) walks the tokens
// once, keeping its slice of the order-2 state in accumulators and writing a snapshot at
// every segment boundary, so the prefix (or suffix) scan over segments is implicit.
// The order-1 state, the denominator matrix Z and the two vector sums are 2*NT*NT + 2*NT
// further 32x32 tiles; they are dealt round-robin to the workgroups of a batch*head (SPW each), and
// inside a workgroup each wavefront adds its quarter of the k-steps, so every workgroup
// does the same amount of work and the grid is exactly (DH / (4*NA)) x bh.  With seg_parallel
// the grid gets a third axis, one walk step per workgroup, and k_state_scan follows (used when
// batch*heads is too small to fill the chip otherwise).  Order 1 has its own kernel, k_build1.
// Replaces the running sums of fastmax_cuda_forward.cu:165-276 (one thread per feature,
// serial over tokens) and the cumsum of materialised outer products of
// fastattention_einops.py:237-248.
template <typename E, int DH, int NA, int TT, int SPW, int KB>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, (NA == 1 && sizeof(E) == 2 && SPW <= 4 && KB < 4 ? 2 : 1)) k_build(BuildArgs<E> A) {
  typedef Mma<E> M;
  typedef typename M::frag frag;
  constexpr int AW = 4 * NA;
  constexpr int NT = DH / 32;                // 32-row tiles per feature axis
  constexpr int PT = TT + M::PAD;
  constexpr int NSMALL = 2 * NT * NT + 2 * NT;
  constexpr int NSTEP = TT / M::KSTEP;
  FM_DYN_SMEM(smem);
  E* s0 = reinterpret_cast<E*>(smem);        // p tile   [DH][PT]
  E* s1 = s0 + DH * PT;                      // r tile   [DH][PT]
  E* s2 = s1 + DH * PT;                      // x rows   [AW][PT]
  E* s3 = s2 + AW * PT;                      // third operand tile [DH][PT] (when zt is given)
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  int grp, bh;
  const int G = FM_GDIM_X;                   // workgroups per batch*head
  fm_xcd_map(G, FM_GDIM_Y, grp, bh);
  const int64_t tb_off = int64_t(bh) * DH * A.npad;
  const int nsteps = (A.mode == FM_WALK_TOTAL) ? 1 : A.nseg - 1;
  if (nsteps <= 0) return;
  E* big = A.big + int64_t(bh) * A.nslots * StateDims<DH>::stride(A.quad != 0);
  E* big2 = A.big2 ? A.big2 + int64_t(bh) * A.nslots * StateDims<DH>::stride(A.quad != 0) : nullptr;
  float* sml = A.small + int64_t(bh) * A.nslots * StateDims<DH>::SMALL;
  const bool has_z = A.zt != nullptr;
  const bool quad = A.quad != 0;

  // small tiles of this workgroup: offsets (elements from s0) of the operand rows in LDS for
  // the A side and the B side (-1: a column of ones)
  int sm_a[SPW], sm_b[SPW], sm_id[SPW];
#pragma unroll
  for (int s = 0; s < SPW; ++s) {
    const int t = grp + s * G;
    sm_id[s] = (t < NSMALL && (quad || t < NT * NT || t >= 2 * NT * NT)) ? t : -1;   // order 1 has no Z
    const int o0 = 0, o1 = DH * PT, o3 = (2 * DH + AW) * PT;
    const int oza = A.za_sel == FM_SRC_P ? o0 : (A.za_sel == FM_SRC_R ? o1 : o3);
    const int ozb = A.zb_sel == FM_SRC_P ? o0 : (A.zb_sel == FM_SRC_R ? o1 : o3);
    int pa = o0, pb = -1;
    if (t < NT * NT) { pa = o0 + 32 * (t / NT) * PT; pb = o1 + 32 * (t % NT) * PT; }                    // order 1
    else if (t < 2 * NT * NT) {
      const int u = t - NT * NT;
      pa = oza + 32 * (u / NT) * PT; pb = ozb + 32 * (u % NT) * PT;                                      // Z
    } else if (t < 2 * NT * NT + NT) pa = oza + 32 * (t - 2 * NT * NT) * PT;                             // va
    else if (t < NSMALL) pa = (A.vb_from_r ? o1 : o0) + 32 * (t - 2 * NT * NT - NT) * PT;                // vb
    sm_a[s] = pa + lr * PT + lh * M::KPL;
    sm_b[s] = pb >= 0 ? pb + lr * PT + lh * M::KPL : -1;
  }

  // the steps of the walk this workgroup takes: all of them in turn, or the one its grid z names.
  // Two cursors run along the walk: `cur` names the token tile being summed, `pf` the tile whose
  // loads are issued next, two tiles ahead (with one tile of lookahead the walk ran at the latency
  // of the memory system: a tile's products take a fraction of a microsecond).
  const int w_end = A.seg_parallel ? FM_BID_Z + 1 : nsteps;
  struct Cursor { int t, w, tb, te, slot; bool valid; };
  auto advance = [&](Cursor& c) {
    c.t += TT;
    if (c.t >= c.te) {
      c.w += 1;
      if (c.w < w_end) { fm_walk_step(A.mode, A.nseg, A.L, A.npad, c.w, c.tb, c.te, c.slot); c.t = c.tb; }
      else c.valid = false;
    }
  };
  Cursor cur;
  cur.w = A.seg_parallel ? FM_BID_Z : 0;
  cur.valid = true;
  fm_walk_step(A.mode, A.nseg, A.L, A.npad, cur.w, cur.tb, cur.te, cur.slot);
  cur.t = cur.tb;
  Cursor pf = cur;
  const int a0 = grp * AW;
  struct Regs { TileRegs<E, DH, TT> p, r, z; TileRegs<E, AW, TT> x; };
  Regs R0, R1;
  auto fetch = [&](Regs& R, const Cursor& c) {
    R.p.load(A.pt + tb_off + c.t, A.npad, tid);
    R.r.load(A.rt + tb_off + c.t, A.npad, tid);
    if (quad) R.x.load(A.xt + tb_off + int64_t(a0) * A.npad + c.t, A.npad, tid);
    if (has_z) R.z.load(A.zt + tb_off + c.t, A.npad, tid);
  };
  fm_f32x16 acc[NA][NT][NT];
  fm_f32x16 sacc[SPW];
#pragma unroll
  for (int i = 0; i < NA; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int k = 0; k < NT; ++k) acc[i][j][k] = fm_zero16();
#pragma unroll
  for (int s = 0; s < SPW; ++s) sacc[s] = fm_zero16();
  // _Float16 walk that has the CU to itself: two LDS buffers of token tiles (see below)
  constexpr bool DB = sizeof(E) == 2 && KB >= 4;
  fetch(R0, pf);
  advance(pf);
  if (!DB && pf.valid) { fetch(R1, pf); advance(pf); }
  // End of a segment: the snapshot of the order-2 slice and the reduced lower-order tiles go to the state of `slot`.
  // mem: LDS that no wavefront reads any more once all of them have arrived here (staging for the stores).
  auto finish_segment = [&](int slot, unsigned char* mem) FM_ALWAYS_INLINE {
#if !defined(FM_HOSTSIM)
    // The accumulators live in the accumulation registers while the products run; without this the
    // compiler copies all of them to vector registers at the end of every tile, ahead of this branch.
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int k = 0; k < NT; ++k)
          if (sizeof(E) == 2 && KB >= 4) asm volatile("" : "+a"(acc[i][j][k]));    // the one-workgroup-per-CU variant
#endif
    if (quad) {
      // snapshot through LDS (the token tiles are spent): accumulators -> staged tiles ->
      // coalesced 16-byte stores; a second pass writes the transposed tiles
      constexpr int SP = DH + M::PAD;
      constexpr int VEC = M::VEC;
      E* stg = reinterpret_cast<E*>(mem);                  // [AW][DH][SP]
      FM_SYNC();
      if (!A.skip_big) {
#pragma unroll
        for (int i = 0; i < NA; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int k = 0; k < NT; ++k)
#pragma unroll
              for (int e = 0; e < 16; ++e)
                stg[((wave * NA + i) * DH + 32 * j + fm_acc_row(e, lh)) * SP + 32 * k + lr] =
                    CE<E>::from(A.coef2 * acc[i][j][k][e]);
        FM_SYNC();
        E* dst = big + int64_t(slot) * StateDims<DH>::BIG + int64_t(a0) * DH * DH;
        for (int c = tid; c < AW * DH * (DH / VEC); c += FM_THREADS) {
          const int row = c / (DH / VEC), col = (c % (DH / VEC)) * VEC;
          *reinterpret_cast<fm_u32x4*>(dst + row * DH + col) = *reinterpret_cast<const fm_u32x4*>(stg + row * SP + col);
        }
        if (big2) FM_SYNC();
      }
      if (big2) {
#pragma unroll
        for (int i = 0; i < NA; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int k = 0; k < NT; ++k)
#pragma unroll
              for (int e = 0; e < 16; ++e)
                stg[((wave * NA + i) * DH + 32 * k + lr) * SP + 32 * j + fm_acc_row(e, lh)] =
                    CE<E>::from(A.coef2b * acc[i][j][k][e]);
        FM_SYNC();
        E* dst2 = big2 + int64_t(slot) * StateDims<DH>::BIG + int64_t(a0) * DH * DH;
        for (int c = tid; c < AW * DH * (DH / VEC); c += FM_THREADS) {
          const int row = c / (DH / VEC), col = (c % (DH / VEC)) * VEC;
          *reinterpret_cast<fm_u32x4*>(dst2 + row * DH + col) = *reinterpret_cast<const fm_u32x4*>(stg + row * SP + col);
        }
      }
    }
    // reduce the four wavefronts' partial lower-order tiles through LDS (the token tiles are
    // spent), RC tiles per pass: every wavefront stores its part of each, then wavefront u adds
    // the four parts of tile u and writes it
    constexpr int RC = SPW < 4 ? SPW : 4;
    float* red = reinterpret_cast<float*>(mem);            // [RC][4 waves][16][64 lanes]
    float* ds = sml + int64_t(slot) * StateDims<DH>::SMALL;
#pragma unroll
    for (int sb = 0; sb < SPW; sb += RC) {
      FM_SYNC();
#pragma unroll
      for (int u = 0; u < RC; ++u)
        if (sb + u < SPW) {
#pragma unroll
          for (int e = 0; e < 16; ++e) red[((u * 4 + wave) * 16 + e) * 64 + lane] = sacc[sb + u][e];
        }
      FM_SYNC();
      const int tl = grp + (sb + wave) * G;
      if (wave < RC && sb + wave < SPW && tl < NSMALL && (quad || tl < NT * NT || tl >= 2 * NT * NT)) {
        float v[16];
#pragma unroll
        for (int e = 0; e < 16; ++e)
          v[e] = red[((wave * 4 + 0) * 16 + e) * 64 + lane] + red[((wave * 4 + 1) * 16 + e) * 64 + lane] +
                 red[((wave * 4 + 2) * 16 + e) * 64 + lane] + red[((wave * 4 + 3) * 16 + e) * 64 + lane];
        fm_put_small<E, DH>(A, big, big2, ds, slot, tl, v, lr, lh);
      }
    }
  };
  if constexpr (DB) {
    // Measured with cycle counters around the phases of the single-buffered loop below (one wavefront per SIMD, so
    // nothing else runs meanwhile): of 4100 cycles per 128-token tile the products and their fragment reads took 40 %,
    // the stores of the next tile into LDS 12 %, issuing its global loads 12 %, the lower-order tiles 8 %, the two
    // barriers and the loop 12 %, the snapshots 16 % -- one after the other.  Here the token tiles have two LDS buffers
    // and two register sets: the stores of tile t + 1 (other buffer) and the global loads of tile t + 2 (other
    // registers) depend on nothing the products of tile t touch, the whole tile is one branch-free block, and the
    // scheduler is told to issue one store or load behind each matrix instruction; one barrier per tile is left.
    static_assert(KB == NSTEP, "all fragments of a tile are requested at once");
    constexpr int TILE_E = (3 * DH + AW) * PT;                 // elements of one buffer: p, r, x, third operand
    unsigned char* const stage_mem = smem + size_t(2) * TILE_E * sizeof(E);
    constexpr size_t RED_BYTES = size_t(SPW < 4 ? SPW : 4) * 4 * 64 * 16 * 4, SNAP_BYTES = size_t(AW) * DH * (DH + M::PAD) * sizeof(E);
    constexpr size_t STAGE_BYTES = RED_BYTES > SNAP_BYTES ? RED_BYTES : SNAP_BYTES;
    auto walk = [&](auto hz_tag) FM_ALWAYS_INLINE {
      constexpr bool HZ = decltype(hz_tag)::value;
      // tile 0 -> buffer 0; tile 1 -> R1
      R0.p.store(s0, PT, tid); R0.r.store(s1, PT, tid); R0.x.store(s2, PT, tid);
      if (HZ) R0.z.store(s3, PT, tid);
      auto fetch_next = [&](Regs& R) FM_ALWAYS_INLINE {
        // the tile `pf` names, or (nothing left to load) the current one again: same instructions either way
        const int t = pf.valid ? pf.t : cur.t;
        R.p.load(A.pt + tb_off + t, A.npad, tid);
        R.r.load(A.rt + tb_off + t, A.npad, tid);
        R.x.load_wrapped(A.xt + tb_off + int64_t(a0) * A.npad + t, A.npad, tid);
        if (HZ) R.z.load(A.zt + tb_off + t, A.npad, tid);
      };
      fetch_next(R1);
      if (pf.valid) advance(pf);
      // eight ones for the lower-order tiles whose second operand is a column of ones: a fragment like any other
      E* const ones_lds = reinterpret_cast<E*>(stage_mem + STAGE_BYTES);
      if (tid < 8) ones_lds[tid] = E(1.0f);
      FM_SYNC();
      // items of a tile: chunk i of p, of r, the x chunk, chunk i of the third operand
      constexpr int NP = TileRegs<E, DH, TT>::N, NITEM = 2 * NP + 1 + (HZ ? NP : 0);
      auto body = [&](const Regs& Rs, Regs& Rf, E* cb, E* nb) FM_ALWAYS_INLINE {
        const E* pb_ = cb + lr * PT + lh * M::KPL;
        const E* rb_ = cb + DH * PT + lr * PT + lh * M::KPL;
        const E* xb_ = cb + 2 * DH * PT + (wave * NA) * PT + lh * M::KPL;
        const int tn = pf.valid ? pf.t : cur.t;     // the tile to load: the one `pf` names, or (none left) the current one again
        frag fb[KB][NT], fp[KB][NT], fx[KB][NA];
        // The fragments of two k-steps are requested ahead of their products (the counter a wavefront waits on
        // for LDS ends at 15 outstanding operations: with all 40 reads of a tile in flight the first product would
        // wait for 26 of them; both walks of a step at the long shape: all at once 1.79 - 1.88 ms, four ahead 1.64,
        // three 1.56, two 1.54).
        constexpr int AHEAD = 2;
        auto frags = [&](int u) FM_ALWAYS_INLINE {
#pragma unroll
          for (int i = 0; i < NA; ++i) fx[u][i] = M::load(xb_ + i * PT + u * M::KSTEP);
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            fp[u][j] = M::load(pb_ + 32 * j * PT + u * M::KSTEP);
            fb[u][j] = M::load(rb_ + 32 * j * PT + u * M::KSTEP);
          }
        };
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) frags(u);
        // the lower-order tiles: this wavefront takes the k-steps wave and wave + 4; their fragments travel with the
        // others (a tile that does not exist for this workgroup is computed on valid operands and never stored)
        constexpr int SK = NSTEP / 4;
        frag sa[SPW][SK], sb[SPW][SK];
#pragma unroll
        for (int u = 0; u < KB; ++u) {
#if !defined(FM_HOSTSIM)
          __builtin_amdgcn_sched_barrier(0);       // the reads, stores and loads below stay with the products of their k-step
#endif
          if (u + AHEAD < KB) frags(u + AHEAD);
          if (u == KB - AHEAD) {
#pragma unroll
            for (int s = 0; s < SPW; ++s)
#pragma unroll
              for (int q = 0; q < SK; ++q) {
                const int ks = wave + 4 * q;
                sa[s][q] = M::load(cb + sm_a[s] + ks * M::KSTEP);
                sb[s][q] = M::load(sm_b[s] >= 0 ? cb + sm_b[s] + ks * M::KSTEP : ones_lds);
              }
          }
#pragma unroll
          for (int i = 0; i < NA; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j) {
              const frag fa = fp[u][j] * fx[u][i];
#pragma unroll
              for (int k = 0; k < NT; ++k) acc[i][j][k] = M::mma(fa, fb[u][k], acc[i][j][k]);
            }
          // this k-step's share of the next tile's stores (registers -> other buffer) and of the loads of the tile after it
#pragma unroll
          for (int it = u * NITEM / KB; it < (u + 1) * NITEM / KB; ++it) {
            if (it < NP) {
              Rs.p.store_part(nb, PT, tid, it);
              Rf.p.load_part(A.pt + tb_off + tn, A.npad, tid, it);
            } else if (it < 2 * NP) {
              Rs.r.store_part(nb + DH * PT, PT, tid, it - NP);
              Rf.r.load_part(A.rt + tb_off + tn, A.npad, tid, it - NP);
            } else if (it == 2 * NP) {
              Rs.x.store_part(nb + 2 * DH * PT, PT, tid, 0);
              Rf.x.load_part(A.xt + tb_off + int64_t(a0) * A.npad + tn, A.npad, tid, 0);
            } else {
              Rs.z.store_part(nb + (2 * DH + AW) * PT, PT, tid, it - 2 * NP - 1);
              Rf.z.load_part(A.zt + tb_off + tn, A.npad, tid, it - 2 * NP - 1);
            }
          }
        }
#pragma unroll
        for (int s = 0; s < SPW; ++s)
#pragma unroll
          for (int q = 0; q < SK; ++q) sacc[s] = M::mma(sa[s][q], sb[s][q], sacc[s]);
#if !defined(FM_HOSTSIM)
        __builtin_amdgcn_sched_barrier(0);
#endif
      };
      auto tail = [&](const E*) FM_ALWAYS_INLINE {
        const bool last = cur.t + TT >= cur.te;
        if (last) finish_segment(cur.slot, stage_mem);
        advance(cur);
        if (pf.valid) advance(pf);
      };
      E* const b0 = s0;
      E* const b1 = s0 + TILE_E;
      while (true) {
        body(R1, R0, b0, b1);
        tail(b0);
        if (!cur.valid) break;
        FM_SYNC();
        body(R0, R1, b1, b0);
        tail(b1);
        if (!cur.valid) break;
        FM_SYNC();
      }
    };
    if (has_z) walk(std::true_type()); else walk(std::false_type());
    return;
  }
  auto stage = [&](Regs& R) FM_ALWAYS_INLINE {
    FM_SYNC();
    R.p.store(s0, PT, tid); R.r.store(s1, PT, tid);
    if (quad) R.x.store(s2, PT, tid);
    if (has_z) R.z.store(s3, PT, tid);
    FM_SYNC();
    if (pf.valid) { fetch(R, pf); advance(pf); }
    const bool last = cur.t + TT >= cur.te;
    const int slot = cur.slot;
    if (quad) {
      const E* pb_ = s0 + lr * PT + lh * M::KPL;
      const E* rb_ = s1 + lr * PT + lh * M::KPL;
      const E* xb_ = s2 + (wave * NA) * PT + lh * M::KPL;
      if (sizeof(E) == 2) {
        // Few k-steps per tile (_Float16): the fragments of KB k-steps are requested from LDS
        // before their first product, so the wavefront waits for LDS NSTEP / KB times per tile
        // (with one k-step of lookahead the walk ran at the LDS latency, not at the MFMA rate).
        // KB = NSTEP needs more than 256 registers: one workgroup per CU.
#pragma unroll
        for (int k0 = 0; k0 < NSTEP; k0 += KB) {
          frag fb[KB][NT], fp[KB][NT], fx[KB][NA];
#pragma unroll
          for (int u = 0; u < KB; ++u) {
#pragma unroll
            for (int j = 0; j < NT; ++j) {
              fb[u][j] = M::load(rb_ + 32 * j * PT + (k0 + u) * M::KSTEP);
              fp[u][j] = M::load(pb_ + 32 * j * PT + (k0 + u) * M::KSTEP);
            }
#pragma unroll
            for (int i = 0; i < NA; ++i) fx[u][i] = M::load(xb_ + i * PT + (k0 + u) * M::KSTEP);
          }
#pragma unroll
          for (int u = 0; u < KB; ++u)
#pragma unroll
            for (int i = 0; i < NA; ++i)
#pragma unroll
              for (int j = 0; j < NT; ++j) {
                const frag fa = fp[u][j] * fx[u][i];
#pragma unroll
                for (int k = 0; k < NT; ++k) acc[i][j][k] = M::mma(fa, fb[u][k], acc[i][j][k]);
              }
        }
      } else {
        // many k-steps per tile (fp32): fragments of k-step ks+1 are fetched while the products of
        // k-step ks are issued
        frag fb[NT], fp[NT], fx[NA];
#pragma unroll
        for (int j = 0; j < NT; ++j) { fb[j] = M::load(rb_ + 32 * j * PT); fp[j] = M::load(pb_ + 32 * j * PT); }
#pragma unroll
        for (int i = 0; i < NA; ++i) fx[i] = M::load(xb_ + i * PT);
#pragma unroll 2
        for (int ks = 0; ks < NSTEP; ++ks) {
          const int kn = (ks + 1 < NSTEP ? ks + 1 : ks) * M::KSTEP;
          frag nb[NT], np[NT], nx[NA];
#pragma unroll
          for (int j = 0; j < NT; ++j) { nb[j] = M::load(rb_ + 32 * j * PT + kn); np[j] = M::load(pb_ + 32 * j * PT + kn); }
#pragma unroll
          for (int i = 0; i < NA; ++i) nx[i] = M::load(xb_ + i * PT + kn);
#pragma unroll
          for (int i = 0; i < NA; ++i) {
#pragma unroll
            for (int j = 0; j < NT; ++j) {
              const frag fa = fp[j] * fx[i];
#pragma unroll
              for (int k = 0; k < NT; ++k) acc[i][j][k] = M::mma(fa, fb[k], acc[i][j][k]);
            }
          }
#pragma unroll
          for (int j = 0; j < NT; ++j) { fb[j] = nb[j]; fp[j] = np[j]; }
#pragma unroll
          for (int i = 0; i < NA; ++i) fx[i] = nx[i];
        }
      }
    }
    // the lower-order tiles: this wavefront takes the k-steps ks = wave (mod 4)
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      if (sm_id[s] >= 0) {
        for (int ks = wave; ks < NSTEP; ks += 4) {
          const frag fa = M::load(s0 + sm_a[s] + ks * M::KSTEP);
          const frag fo = sm_b[s] >= 0 ? M::load(s0 + sm_b[s] + ks * M::KSTEP) : M::splat(E(1.0f));
          sacc[s] = M::mma(fa, fo, sacc[s]);
        }
      }
    }
    if (last) finish_segment(slot, smem);
    advance(cur);
  };
  while (true) {
    stage(R0);
    if (!cur.valid) break;
    stage(R1);
    if (!cur.valid) break;
  }
}

// k_build1: the order-1 states (the D x D sum and the two vector sums, no Z) of one walk step per
// workgroup; grid (1, bh, steps), k_state_scan follows when there are several steps.  The sums are
// 8 tiles for D = 64, far too little work per token tile to pay for staging and barriers: each
// wavefront takes a quarter of the step's tokens and loads its MFMA fragments straight from the
// transposed operands (16 bytes per lane, four k-steps in flight), and the four partial sums meet
// in LDS once at the end.  Needs (te - tb) to be a multiple of 4 * 4 * KSTEP tokens (segments and
// padded lengths are multiples of 256).
template <typename E, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, 2) k_build1(BuildArgs<E> A) {
  typedef Mma<E> M;
  typedef typename M::frag frag;
  constexpr int NT = DH / 32, NTILE = NT * NT + 2 * NT, UB = 4;
  FM_DYN_SMEM(smem);
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  const int bh = FM_BID_Y;
  int tb, te, slot;
  fm_walk_step(A.mode, A.nseg, A.L, A.npad, FM_BID_Z, tb, te, slot);
  E* big = A.big + int64_t(bh) * A.nslots * StateDims<DH>::stride(A.quad != 0);
  E* big2 = A.big2 ? A.big2 + int64_t(bh) * A.nslots * StateDims<DH>::stride(A.quad != 0) : nullptr;
  float* ds = A.small + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL;
  const int per_wave = (te - tb) / 4;                  // tokens of this wavefront
  const int64_t row = (int64_t(bh) * DH + lr) * A.npad + tb + wave * per_wave + lh * M::KPL;
  const E* pp = A.pt + row;
  const E* rp = A.rt + row;
  const bool has_z = A.zt != nullptr;
  const E* zp = has_z ? A.zt + row : pp;
  const int za = A.za_sel;
  const bool vb_r = A.vb_from_r != 0;
  const int64_t tile = int64_t(32) * A.npad;           // 32 feature rows further
  fm_f32x16 acc[NTILE];
#pragma unroll
  for (int i = 0; i < NTILE; ++i) acc[i] = fm_zero16();
  const frag ones = M::splat(E(1.0f));
  for (int t = 0; t < per_wave; t += UB * M::KSTEP) {
    frag fp[UB][NT], fr[UB][NT], fz[UB][NT];
#pragma unroll
    for (int u = 0; u < UB; ++u)
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        fp[u][j] = M::load(pp + j * tile + t + u * M::KSTEP);
        fr[u][j] = M::load(rp + j * tile + t + u * M::KSTEP);
        fz[u][j] = has_z ? M::load(zp + j * tile + t + u * M::KSTEP) : fp[u][j];
      }
#pragma unroll
    for (int u = 0; u < UB; ++u) {
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i * NT + j] = M::mma(fp[u][i], fr[u][j], acc[i * NT + j]);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const frag fa = za == FM_SRC_P ? fp[u][j] : (za == FM_SRC_R ? fr[u][j] : fz[u][j]);
        acc[NT * NT + j] = M::mma(fa, ones, acc[NT * NT + j]);
        acc[NT * NT + NT + j] = M::mma(vb_r ? fr[u][j] : fp[u][j], ones, acc[NT * NT + NT + j]);
      }
    }
  }
  // the four wavefronts' partial tiles meet in LDS, RC tiles per pass; wavefront u adds and writes tile u
  constexpr int RC = 4;
  float* red = reinterpret_cast<float*>(smem);         // [RC][4 waves][16][64 lanes]
#pragma unroll
  for (int sb = 0; sb < NTILE; sb += RC) {
    if (sb) FM_SYNC();
#pragma unroll
    for (int u = 0; u < RC; ++u)
      if (sb + u < NTILE) {
#pragma unroll
        for (int e = 0; e < 16; ++e) red[((u * 4 + wave) * 16 + e) * 64 + lane] = acc[sb + u][e];
      }
    FM_SYNC();
    const int i = sb + wave;
    if (i < NTILE) {
      float v[16];
#pragma unroll
      for (int e = 0; e < 16; ++e)
        v[e] = red[((wave * 4 + 0) * 16 + e) * 64 + lane] + red[((wave * 4 + 1) * 16 + e) * 64 + lane] +
               red[((wave * 4 + 2) * 16 + e) * 64 + lane] + red[((wave * 4 + 3) * 16 + e) * 64 + lane];
      fm_put_small<E, DH>(A, big, big2, ds, slot, i < NT * NT ? i : i + NT * NT, v, lr, lh);
    }
  }
}

// k_build1_seg: the same sums for a walk of several steps (one workgroup per segment and
// batch*head, k_state_scan follows).  A lane's MFMA fragment is 16 bytes of one feature row of a
// transposed operand, and the rows lie a power of two apart: loaded straight from memory, the 32
// rows of one load instruction queue up behind one another (measured on MI355X: the loads alone
// were 145 of the 170 us of a launch over 16 x 65536 tokens).  So the workgroup stages the operand
// tiles of 128 tokens through LDS with whole 256-byte row pieces per 16 lanes (the next tile
// travels global memory -> registers meanwhile), and the tiles of the sums, not the tokens, are
// dealt to the wavefronts: wavefront w sums tiles w, w + 4, .. (for D = 64 one tile of the D x D
// sum and one vector-sum tile) over all tokens, so no partial sums meet anywhere.
// Needs (te - tb) to be a multiple of 128 tokens.
template <typename E, int DH> struct Build1Cfg {
  static constexpr int TT = 128, PT = TT + Mma<E>::VEC;
  static constexpr size_t lds_bytes(bool has_z) { return size_t(has_z ? 3 : 2) * DH * PT * sizeof(E); }
};

template <typename E, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS) k_build1_seg(BuildArgs<E> A) {
  typedef Mma<E> M;
  typedef typename M::frag frag;
  constexpr int NT = DH / 32, NTILE = NT * NT + 2 * NT, NS = (NTILE + 3) / 4;
  constexpr int TT = Build1Cfg<E, DH>::TT, PT = Build1Cfg<E, DH>::PT;
  FM_DYN_SMEM(smem);
  E* Lp = reinterpret_cast<E*>(smem);                  // [DH][PT] each
  E* Lr = Lp + DH * PT;
  E* Lz = Lr + DH * PT;                                // only there (and only used) with a third operand
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  const int bh = FM_BID_Y;
  int tb, te, slot;
  fm_walk_step(A.mode, A.nseg, A.L, A.npad, FM_BID_Z, tb, te, slot);
  E* big = A.big + int64_t(bh) * A.nslots * StateDims<DH>::stride(A.quad != 0);
  E* big2 = A.big2 ? A.big2 + int64_t(bh) * A.nslots * StateDims<DH>::stride(A.quad != 0) : nullptr;
  float* ds = A.small + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL;
  const bool has_z = A.zt != nullptr && A.za_sel == FM_SRC_Z;
  const int64_t base = int64_t(bh) * DH * A.npad;
  const E* gp = A.pt + base;
  const E* gr = A.rt + base;
  const E* gz = has_z ? A.zt + base : gp;
  const E* va_src = A.za_sel == FM_SRC_P ? Lp : (A.za_sel == FM_SRC_R ? Lr : Lz);
  const E* vb_src = A.vb_from_r ? Lr : Lp;
  const E* la[NS];
  const E* lb[NS];                                      // null: a vector sum (the B operand is all ones)
  int tl[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int t = wave + 4 * s;
    const int frag_off = lr * PT + lh * M::KPL;
    tl[s] = t;
    la[s] = Lp + frag_off; lb[s] = nullptr;
    if (t < NT * NT) { la[s] = Lp + (t / NT) * 32 * PT + frag_off; lb[s] = Lr + (t % NT) * 32 * PT + frag_off; }
    else if (t < NT * NT + NT) la[s] = va_src + (t - NT * NT) * 32 * PT + frag_off;
    else if (t < NTILE) la[s] = vb_src + (t - NT * NT - NT) * 32 * PT + frag_off;
  }
  fm_f32x16 acc[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) acc[s] = fm_zero16();
  const frag ones = M::splat(E(1.0f));
  TileRegs<E, DH, TT> rp, rr, rz;
  auto fetch = [&](int t0) {                            // global memory -> registers
    rp.load(gp + t0, A.npad, tid);
    rr.load(gr + t0, A.npad, tid);
    if (has_z) rz.load(gz + t0, A.npad, tid);
  };
  fetch(tb);
  for (int t0 = tb; t0 < te; t0 += TT) {
    if (t0 != tb) FM_SYNC();                            // the previous tile has been read
    rp.store(Lp, PT, tid);
    rr.store(Lr, PT, tid);
    if (has_z) rz.store(Lz, PT, tid);
    if (t0 + TT < te) fetch(t0 + TT);
    FM_SYNC();
#pragma unroll
    for (int s = 0; s < NS; ++s)
      if (tl[s] < NTILE) {
#pragma unroll 8
        for (int k = 0; k < TT; k += M::KSTEP)
          acc[s] = M::mma(M::load(la[s] + k), lb[s] ? M::load(lb[s] + k) : ones, acc[s]);
      }
  }
#pragma unroll
  for (int s = 0; s < NS; ++s)
    if (tl[s] < NTILE) {
      float v[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) v[e] = acc[s][e];
      fm_put_small<E, DH>(A, big, big2, ds, slot, tl[s] < NT * NT ? tl[s] : tl[s] + NT * NT, v, lr, lh);
    }
}

// k_build1_rows: k_build1_seg for element types with a transposing LDS read, from the ROW-major
// operand copies the token kernels stream anyway ([token][feature], a segment's 128 tokens are one
// contiguous 16 KB piece): the tiles are staged as they lie and every MFMA fragment (tokens along
// the contraction axis) is a transposing read, so no transposed copy of any operand has to exist
// for an order-1 problem.  The transposing read hands a lane the 16 tokens of a k-step in `tperm`
// order, which is the order the per-token weights `cw` are stored in, so a weighted vector sum
// (sum_t cw_t p_t: the third operand of the backward's walk) takes its B fragment straight from
// the staged weights.  Tiles are dealt to the wavefronts as in k_build1_seg.
template <typename E, int DH> struct Build1RowsCfg {
  static constexpr int TT = 128, PQ = DH + Mma<E>::PAD;
  static constexpr size_t lds_bytes() { return (size_t(2) * TT * PQ + TT) * sizeof(E); }
};

template <typename E, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_THREADS) k_build1_rows(BuildArgs<E> A) {
  typedef Mma<E> M;
  typedef typename M::frag frag;
  constexpr int NT = DH / 32, NTILE = NT * NT + 2 * NT, NS = (NTILE + 3) / 4;
  constexpr int TT = Build1RowsCfg<E, DH>::TT, PQ = Build1RowsCfg<E, DH>::PQ;
  FM_DYN_SMEM(smem);
  E* Lp = reinterpret_cast<E*>(smem);                  // [TT][PQ] each
  E* Lr = Lp + TT * PQ;
  E* Lc = Lr + TT * PQ;                                // [TT] weights
  const int tid = FM_TID_X, lane = tid & 63, lh = lane >> 5;
  const int wave = FM_UNIFORM(tid >> 6);
  const int bh = FM_BID_Y;
  int tb, te, slot;
  fm_walk_step(A.mode, A.nseg, A.L, A.npad, FM_BID_Z, tb, te, slot);
  E* big = A.big + int64_t(bh) * A.nslots * StateDims<DH>::stride(A.quad != 0);
  E* big2 = A.big2 ? A.big2 + int64_t(bh) * A.nslots * StateDims<DH>::stride(A.quad != 0) : nullptr;
  float* ds = A.small + (int64_t(bh) * A.nslots + slot) * StateDims<DH>::SMALL;
  const bool has_w = A.cw != nullptr;
  const E* gp = A.pr + int64_t(bh) * A.npad * DH;
  const E* gr = A.rr + int64_t(bh) * A.npad * DH;
  const float* gc = has_w ? A.cw + int64_t(bh) * A.npad : nullptr;
  // the tiles of this wavefront: A operand (tile, feature offset), B operand (tile or null = weights / ones)
  const E* ta[NS]; const E* tbt[NS];
  int fa_off[NS], fb_off[NS], tl[NS];
  bool wsum[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int t = wave + 4 * s;
    tl[s] = t;
    ta[s] = Lp; tbt[s] = nullptr; fa_off[s] = 0; fb_off[s] = 0; wsum[s] = false;
    if (t < NT * NT) { fa_off[s] = 32 * (t / NT); tbt[s] = Lr; fb_off[s] = 32 * (t % NT); }
    else if (t < NT * NT + NT) {
      fa_off[s] = 32 * (t - NT * NT);
      if (A.za_sel == FM_SRC_R) ta[s] = Lr;
      wsum[s] = A.za_sel == FM_SRC_Z;                   // sum_t cw_t p_t
    } else if (t < NTILE) {
      fa_off[s] = 32 * (t - NT * NT - NT);
      if (A.vb_from_r) ta[s] = Lr;
    }
  }
  fm_f32x16 acc[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) acc[s] = fm_zero16();
  const frag ones = M::splat(E(1.0f));
  TileRegs<E, TT, DH> rp, rr;
  float creg = 0.f;
  auto fetch = [&](int t0) {                            // global memory -> registers
    rp.load(gp + int64_t(t0) * DH, DH, tid);
    rr.load(gr + int64_t(t0) * DH, DH, tid);
    if (has_w && tid < TT) creg = gc[t0 + tid];
  };
  fetch(tb);
  for (int t0 = tb; t0 < te; t0 += TT) {
    if (t0 != tb) FM_SYNC();                            // the previous tile has been read
    rp.store(Lp, PQ, tid);
    rr.store(Lr, PQ, tid);
    if (has_w && tid < TT) Lc[tid] = CE<E>::from(creg);
    if (t0 + TT < te) fetch(t0 + TT);
    FM_SYNC();
#pragma unroll
    for (int s = 0; s < NS; ++s)
      if (tl[s] < NTILE) {
#pragma unroll 4
        for (int k = 0; k < TT; k += M::KSTEP) {
          const frag fa = M::load_tr(ta[s], PQ, k, fa_off[s], lane);
          const frag fb = tbt[s] ? M::load_tr(tbt[s], PQ, k, fb_off[s], lane)
                                 : (wsum[s] ? M::load_perm(Lc + k, 0, lh) : ones);
          acc[s] = M::mma(fa, fb, acc[s]);
        }
      }
  }
  const int lr = lane & 31;
#pragma unroll
  for (int s = 0; s < NS; ++s)
    if (tl[s] < NTILE) {
      float v[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) v[e] = acc[s][e];
      fm_put_small<E, DH>(A, big, big2, ds, slot, tl[s] < NT * NT ? tl[s] : tl[s] + NT * NT, v, lr, lh);
    }
}

// ------------------------------------------------------------------------------
// k_state_scan: turns per-segment sums (k_build with seg_parallel) into the states the readers
// expect: slot s becomes the sum over the walk up to and including its own step.  Elementwise
// over the order-1 slab of `big` (and of `big2`), over the order-2 slabs too when quad, and over
// the vector sums (and Z when quad) of `small`; the running sum is kept in fp32.
// ------------------------------------------------------------------------------
// Running sums over the walk of the 16 bytes at p: `stride` elements lie between the slots of two
// consecutive steps.  32 steps are loaded before any is added and stored, so the chain of
// dependent memory round trips is a 32nd as long as the walk (the launch is a few dozen
// workgroups, so the round trips, not the bytes, set its time).
template <typename T> FM_DEVICE void fm_scan_run(T* p, int64_t stride, int nsteps) {
  constexpr int UB = 32, VE = 16 / sizeof(T);
  float run[VE];
#pragma unroll
  for (int i = 0; i < VE; ++i) run[i] = 0.f;
  for (int w0 = 0; w0 < nsteps; w0 += UB) {
    fm_u32x4 raw[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u)
      if (w0 + u < nsteps) raw[u] = *reinterpret_cast<const fm_u32x4*>(p + (w0 + u) * stride);
#pragma unroll
    for (int u = 0; u < UB; ++u)
      if (w0 + u < nsteps) {
        T v[VE];
        __builtin_memcpy(v, &raw[u], 16);
#pragma unroll
        for (int i = 0; i < VE; ++i) { run[i] += float(v[i]); v[i] = CE<T>::from(run[i]); }
        fm_u32x4 out;
        __builtin_memcpy(&out, v, 16);
        *reinterpret_cast<fm_u32x4*>(p + (w0 + u) * stride) = out;
      }
  }
}

// grid (ceil(items / FM_SCAN_THREADS), bh); an item is 16 bytes of one state array.
#define FM_SCAN_THREADS 64
template <typename E, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(FM_SCAN_THREADS) k_state_scan(E* FM_RESTRICT big, E* FM_RESTRICT big2, float* FM_RESTRICT small,
                                                  int nslots, int nsteps, int mode, int nseg, int quad) {
  constexpr int VE = 16 / sizeof(E);
  const int bh = FM_BID_Y;
  const int64_t nbig = (quad ? int64_t(DH + 1) * DH * DH : int64_t(DH) * DH) / VE;   // items of big
  const int64_t first = 0;                                      // order 1: the slot is the order-1 slab alone
  const int64_t sstride = StateDims<DH>::stride(quad != 0);
  const int64_t sfirst = quad ? 0 : int64_t(DH) * DH;           // order 1 has no Z: only the two vectors
  const int64_t nsmall = (StateDims<DH>::SMALL - sfirst) / 4;
  const int64_t nb2 = nbig * (big2 ? 2 : 1);
  const int64_t i = int64_t(FM_BID_X) * FM_SCAN_THREADS + FM_TID_X;
  if (i >= nb2 + nsmall) return;
  // the slot k_build's step w writes is slot0 + w * dir
  const int slot0 = mode == FM_WALK_PREFIX ? 1 : nseg - 2;
  const int dir = mode == FM_WALK_PREFIX ? 1 : -1;
  if (i < nb2) {
    E* b = (i < nbig ? big : big2) + (int64_t(bh) * nslots + slot0) * sstride + first + (i < nbig ? i : i - nbig) * VE;
    fm_scan_run<E>(b, int64_t(dir) * sstride, nsteps);
  } else {
    float* sp = small + (int64_t(bh) * nslots + slot0) * StateDims<DH>::SMALL + sfirst + (i - nb2) * 4;
    fm_scan_run<float>(sp, int64_t(dir) * StateDims<DH>::SMALL, nsteps);
  }
}

// ------------------------------------------------------------------------------
// Shared pieces of the token-side kernels
// ------------------------------------------------------------------------------
// LDS sizes (in elements of E) used by k_pv / k_ds; the host computes the dynamic LDS
// bytes from the same struct.
// Stream tokens per stage of the dense loops of the _Float16 token kernels.  k_ds stages two row
// tiles only (its transposed fragments come from transposing LDS reads), so 64-token stages cost it
// no occupancy and halve its barriers (dQ 0.117 -> 0.114 ms at B*H = 32, N = 4096 on MI355X); k_pv
// measured slower with them (0.092 vs 0.087 ms).
template <typename E, int DH, int QT>
struct TokCfg {
  typedef Mma<E> M;
  static constexpr int NT = DH / 32;
  static constexpr int NKS = DH / M::KSTEP;         // k-steps over a feature axis
  static constexpr int QW = 4 * QT * 32;            // tokens per workgroup
  static constexpr int PQ = DH + M::PAD;            // pitch of row-major token tiles
  static constexpr int PS = DH + M::PAD;            // pitch of state rows
  // _Float16, QT = 1: one tile per wavefront, small slabs and stages, so that four (k_pv) or three
  // (k_ds) workgroups share a CU: 12 to 16 wavefronts hide each other's LDS and MFMA latency.  On
  // MI355X at B*H = 32, N = 4096, D = 64 this measured faster on dense tiles than two tiles per
  // wavefront at two workgroups per CU (0.47 vs 0.56 ms for the four kernels together).
  // _Float16, QT = 2: two tiles per wavefront share every state fragment read from LDS and halve
  // the state bytes staged per token; used by k_ds when there are states to read (dQ + dK
  // 0.20 vs 0.23 ms at the same shape with 1024-token segments).
  // Heads wider than 64 (DH = 128, _Float16, dense tiles only: see FM_WIDE_HEAD in fastmax_api.hip) hold twice the
  // accumulators and own fragments: two workgroups per CU for k_pv, one for k_ds.
  static constexpr bool WIDE = DH > 64;
  static constexpr int OCC_PV = WIDE ? 2 : (sizeof(E) == 2 ? (QT == 1 ? 4 : 2) : 1);   // workgroups per CU the kernels are sized for
  static constexpr int OCC_DS = WIDE ? 1 : (sizeof(E) == 2 ? (QT == 1 ? 3 : 2) : 1);
  static constexpr int OCC_DV = WIDE ? 1 : 2;
  static constexpr int SA = sizeof(E) == 2 ? QT : 2;                      // values of a per state slab
  static constexpr int KT_PV = sizeof(E) == 2 ? 32 : 64;   // stream tokens per stage of the dense loop, k_pv
  static constexpr int KT_DS = 64;                        //                                           k_ds
  // the dK + dV pass runs two workgroups per CU whatever its stages are, and 64-token stages
  // halve its barriers (0.163 vs 0.173 ms at the shape above)
  static constexpr int KT_DV = 64;                        //                                           k_ds with dV
  static constexpr int PV_PV = KT_PV + M::PAD;      // pitch of the transposed token tiles
  static constexpr int PV_DS = KT_DS + M::PAD;
  static constexpr int PV_DV = KT_DV + M::PAD;
  static constexpr int NZ = sizeof(E) == 2 ? 2 : 1; // hi/lo split of fp32 denominators
  static constexpr int SLAB = SA * DH * PS;         // elements per slab buffer
  // the symmetric readout's narrow blocks stage twice the values of a in compact rows (see SymBlk)
  static constexpr int SLAB_SYM = (sizeof(E) == 2 && 2 * SA * DH * (DH / 2 + M::PAD) > SLAB) ? 2 * SA * DH * (DH / 2 + M::PAD) : SLAB;
  static constexpr int PV_STAGE = M::HAS_TR ? 2 * KT_PV * PQ : KT_PV * PQ + DH * PV_PV;   // k_pv: two row tiles, or stream rows + stream transposed
  // c values of a stage: KT compute-type elements, or KT floats (the completed-square kernels stage -c in fp32)
  static constexpr int DS_STAGE = 2 * KT_DS * PQ + (M::HAS_TR ? 0 : DH * PV_DS) + (M::HAS_TR ? 2 : 1) * KT_DS;   // k_ds: two row tiles, (transposed tile,) c values
  // k_ds with dV: two row tiles and the c values; the transposed fragments come from the row tiles
  // through transposing LDS reads where the type has them, from two more (transposed) tiles otherwise
  static constexpr int DV_STAGE = 2 * KT_DV * PQ + (M::HAS_TR ? 0 : 2 * DH * PV_DV) + (M::HAS_TR ? 2 : 1) * KT_DV;
  static constexpr int DS_NBUF = sizeof(E) == 2 ? 2 : 1;
};

// Moment readout, transposed:  acc[j][ct] (rows c, column = token of tile j) +=
//   sum_{a, b} T[a][c][b] * x_a(token) * y_b(token)        a < DH
//   sum_b      T[DH][c][b] * y_b(token)                    a = DH
// xs: row-major token tile in LDS (pitch PQ) supplying x; yb[j][ks]: B fragments of y.
// slab: two buffers of SA*DH*PS elements.  All 256 threads must call this.
// The A fragments of step i+1 are fetched from LDS before the products of step i are
// issued, so a single wavefront per SIMD keeps the matrix pipe fed.
// TRA: the slabs lie transposed in memory, T[a][b][c] (rows b, columns c): the A fragments are read out of the
// staged slab with transposing LDS reads, and yb must then hold y in the k order those reads deliver (16 s +
// 4 lh + {0..3}, 16 s + 8 + 4 lh + {0..3}: Mma::load_nat_perm).  This is how dQ reads the forward's own
// (k, v, k) state, whose slab a is [v][k]: U[a][v][k] = sum k_a v k is symmetric in its two key indices, so it is
// the transposed slab of the (k, k, v) state dQ contracts.  xscale: factor on x (the order-2 part only).
template <typename E, int DH, int QT, int NACC, bool TRA = false>
FM_DEVICE void fm_readout(const E* FM_RESTRICT state, bool quad, const E* xs, const int* xrow,
                          const typename Mma<E>::frag (*yb)[TokCfg<E, DH, QT>::NKS],
                          E* slab, fm_f32x16 (*acc)[NACC], int tid, float xscale = 1.0f) {
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  typedef typename M::frag frag;
  const int lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int a_begin = quad ? 0 : DH;
  const E xs_f = CE<E>::from(xscale);
  // TRA: the lane's row (4 lh + s4 inside a k-step) and its columns inside the swizzled rows, per row tile; which half
  // of a row the columns lie in depends on bit 1 of the row, i.e. of s4 alone
  int tr_base[C::NT];
  {
    const int s4 = (lane & 15) >> 2, q = lane & 3, half16 = (lane >> 4) & 1;
#pragma unroll
    for (int ct = 0; ct < C::NT; ++ct)
      tr_base[ct] = (4 * lh + s4) * DH + ((32 * ct + 16 * half16 + 4 * q) ^ (((s4 >> 1) & 1) * (DH / 2)));
  }
  TileRegs<E, C::SA * DH, DH> regs;
  // `state` points at the first slab to read (T[0] with order-2 states, else the order-1 slab)
  regs.load(state, DH, tid);                                  // rows [a][c] are contiguous
  int buf = 0;
  const int lane_off = lr * C::PS + lh * M::KPL;
  for (int as = a_begin; as <= DH; as += C::SA) {
    E* sb = slab + buf * C::SLAB;
    if constexpr (TRA) {
      // Rows without padding, the 16-byte chunks of rows 2, 3 (mod 4) exchanged between the two halves of the row: the
      // four rows a transposing read touches per half-wavefront then lie in four different quarters of the banks
      // (with the padded pitch rows r and r + 2 share banks and every such read takes twice as long).
      typedef TileRegs<E, C::SA * DH, DH> TR_;
#pragma unroll
      for (int i = 0; i < TR_::N; ++i) {
        const int c = tid + FM_THREADS * i;
        if (TR_::TOTAL % FM_THREADS == 0 || c < TR_::TOTAL) {
          const int row = c / TR_::CPR, ch = c % TR_::CPR;
          *reinterpret_cast<fm_u32x4*>(sb + row * DH + ((ch ^ (((row >> 1) & 1) * (TR_::CPR / 2))) * TR_::VEC)) = regs.r[i];
        }
      }
    } else {
      regs.store(sb, C::PS, tid);
    }
    FM_SYNC();
    if (as + C::SA <= DH) regs.load(state + int64_t(as + C::SA - a_begin) * DH * DH, DH, tid);
    const int na = (as + C::SA <= DH) ? C::SA : (DH + 1 - as);
    const E* sl = sb + lane_off;
    // fragment (value al of the slab, row tile ct, k-step ks)
    auto afrag = [&](int al, int ct, int ks) FM_ALWAYS_INLINE {
      if constexpr (TRA) {
        // Mma::load_tr on the swizzled rows; the lane's part of the address was formed once (tr_base)
        const E* p = sb + tr_base[ct] + (al * DH + ks * M::KSTEP) * DH;
        const fm_half4 lo = fm_lds_tr4(p), hi = fm_lds_tr4(p + 8 * DH);
        frag r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return r;
      } else return M::load(sl + (al * DH + 32 * ct) * C::PS + ks * M::KSTEP);
    };
    frag fa[C::NT];
#pragma unroll
    for (int ct = 0; ct < C::NT; ++ct) fa[ct] = afrag(0, ct, 0);
    // the own tokens' x_a: the value for the next a is read from LDS while this one's products run
    E xv[QT];
#pragma unroll
    for (int j = 0; j < QT; ++j) xv[j] = (as < DH) ? xs[xrow[j] * C::PQ + as] * xs_f : E(1.0f);
    for (int al = 0; al < na; ++al) {
      const int a = as + al;
      frag xr[QT];
#pragma unroll
      for (int j = 0; j < QT; ++j) xr[j] = M::splat(xv[j]);
      const int an = (al + 1 < na) ? a + 1 : a;        // re-reads a valid element at the end of a slab
#pragma unroll
      for (int j = 0; j < QT; ++j) xv[j] = (an < DH) ? xs[xrow[j] * C::PQ + an] * xs_f : E(1.0f);
#pragma unroll
      for (int ks = 0; ks < C::NKS; ++ks) {
        // prefetch the fragments of the next (a, k-step); the last one of a slab re-reads a valid row
        const int nks = (ks + 1 < C::NKS) ? ks + 1 : 0;
        const int nal = (ks + 1 < C::NKS) ? al : (al + 1 < na ? al + 1 : al);
        frag fn[C::NT];
#pragma unroll
        for (int ct = 0; ct < C::NT; ++ct) fn[ct] = afrag(nal, ct, nks);
#pragma unroll
        for (int j = 0; j < QT; ++j) {
          const frag fb = yb[j][ks] * xr[j];
#pragma unroll
          for (int ct = 0; ct < C::NT; ++ct) acc[j][ct] = M::mma(fa[ct], fb, acc[j][ct]);
        }
#pragma unroll
        for (int ct = 0; ct < C::NT; ++ct) fa[ct] = fn[ct];
      }
    }
    buf ^= 1;
  }
  FM_SYNC();
}

// The same readout when x and y are one vector and T[a][c][b] = T[b][c][a] (the forward's (k, v, k) sums read with
// q, and the (q, gh, q) sums dV reads with k): sum_{a, b} = the 16 x 16 blocks on the diagonal of (a, b) once plus
// twice the blocks above it, so a value of `a` in block KB meets the k-steps KB .. NKS - 1 only -- 10 of 16
// products and 10 of 16 bytes of every slab, whose unused columns are neither loaded nor staged.
// Blocks of half the full width or less hold twice the values of `a` per slab, in compact rows (as many bytes per
// stage as the full-width slabs: the barrier and the slab's way into LDS are paid per stage).
constexpr int FM_SYM_BLOCK = 16;
template <typename E, int DH, int QT, int KB> struct SymBlk {
  typedef TokCfg<E, DH, QT> C;
  static constexpr int C0 = KB * FM_SYM_BLOCK, W = DH - C0;             // first column and columns met
  static constexpr bool TALL = sizeof(E) == 2 && 2 * W <= DH;
  static constexpr int SAB = TALL ? 2 * C::SA : C::SA;                  // values of a per slab
  static constexpr int PSB = TALL ? W + Mma<E>::PAD : C::PS;            // row pitch of the staged slab
  static constexpr int OFF = TALL ? 0 : C0;                             // where column C0 lies in a staged row
  static_assert(SAB * DH * PSB <= C::SLAB_SYM, "a slab fits its buffer");
};
// products of one staged slab: values as .. as + na - 1 of a (rows [al][c] at pitch PSB, column C0 at OFF)
template <typename E, int DH, int QT, int NACC, int KB, int PSB, int OFF>
FM_DEVICE void fm_readout_products(const E* sb, const E* xs, const int* xrow, int as, int na, bool ones,
                                   const typename Mma<E>::frag (*yb)[TokCfg<E, DH, QT>::NKS], fm_f32x16 (*acc)[NACC],
                                   int lr, int lh) {
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  typedef typename M::frag frag;
  constexpr int KPB = FM_SYM_BLOCK / M::KSTEP;       // k-steps per block of (a, b)
  constexpr int K0 = KB * KPB;                       // first k-step met
  const E* sl = sb + lr * PSB + lh * M::KPL + OFF - K0 * M::KSTEP;      // column col of row 0 of the lane: sl + col
  frag fa[C::NT];
#pragma unroll
  for (int ct = 0; ct < C::NT; ++ct) fa[ct] = M::load(sl + (32 * ct) * PSB + K0 * M::KSTEP);
  E xv[QT];
#pragma unroll
  for (int j = 0; j < QT; ++j) xv[j] = ones ? E(1.0f) : xs[xrow[j] * C::PQ + as];
  for (int al = 0; al < na; ++al) {
    frag xr[QT], xr2[QT];
#pragma unroll
    for (int j = 0; j < QT; ++j) { xr[j] = M::splat(xv[j]); xr2[j] = ones ? xr[j] : xr[j] + xr[j]; }
    const int an = (al + 1 < na) ? as + al + 1 : as + al;
#pragma unroll
    for (int j = 0; j < QT; ++j) xv[j] = ones ? E(1.0f) : xs[xrow[j] * C::PQ + an];
#pragma unroll
    for (int ks = K0; ks < C::NKS; ++ks) {
      const int nks = (ks + 1 < C::NKS) ? ks + 1 : K0;
      const int nal = (ks + 1 < C::NKS) ? al : (al + 1 < na ? al + 1 : al);
      frag fn[C::NT];
#pragma unroll
      for (int ct = 0; ct < C::NT; ++ct) fn[ct] = M::load(sl + (nal * DH + 32 * ct) * PSB + nks * M::KSTEP);
#pragma unroll
      for (int j = 0; j < QT; ++j) {
        const frag fb = yb[j][ks] * (ks < K0 + KPB ? xr[j] : xr2[j]);
#pragma unroll
        for (int ct = 0; ct < C::NT; ++ct) acc[j][ct] = M::mma(fa[ct], fb, acc[j][ct]);
      }
#pragma unroll
      for (int ct = 0; ct < C::NT; ++ct) fa[ct] = fn[ct];
    }
  }
}

template <typename E, int DH, int QT, int NACC, int KB>
FM_DEVICE void fm_readout_sym_block(const E* FM_RESTRICT state,
                                    TileRegs<E, SymBlk<E, DH, QT, KB>::SAB * DH, SymBlk<E, DH, QT, KB>::W>& cur,
                                    const E* xs, const int* xrow, const typename Mma<E>::frag (*yb)[TokCfg<E, DH, QT>::NKS],
                                    E* slab, fm_f32x16 (*acc)[NACC], int tid, int& buf) {
  typedef TokCfg<E, DH, QT> C;
  typedef Mma<E> M;
  typedef SymBlk<E, DH, QT, KB> B;
  constexpr int C0 = B::C0, A_END = C0 + FM_SYM_BLOCK;
  constexpr bool LASTB = A_END == DH;
  static_assert(FM_SYM_BLOCK % B::SAB == 0 && FM_SYM_BLOCK % M::KSTEP == 0 && DH % FM_SYM_BLOCK == 0, "whole slabs and k-steps per block");
  typedef SymBlk<E, DH, QT, LASTB ? 0 : KB + 1> BN;
  const int lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  // after the last block: the order-1 slab (DH rows, every column)
  TileRegs<E, LASTB ? DH : BN::SAB * DH, LASTB ? DH : BN::W> nxt;
  for (int as = C0; as < A_END; as += B::SAB) {
    E* sb = slab + buf * C::SLAB_SYM;
    cur.store(sb + B::OFF, B::PSB, tid);
    FM_SYNC();
    if (as + B::SAB < A_END) cur.load(state + int64_t(as + B::SAB) * DH * DH + C0, DH, tid);
    else nxt.load(state + int64_t(as + B::SAB) * DH * DH + (LASTB ? 0 : A_END), DH, tid);
    fm_readout_products<E, DH, QT, NACC, KB, B::PSB, B::OFF>(sb, xs, xrow, as, B::SAB, false, yb, acc, lr, lh);
    buf ^= 1;
  }
  if constexpr (!LASTB) {
    fm_readout_sym_block<E, DH, QT, NACC, KB + 1>(state, nxt, xs, xrow, yb, slab, acc, tid, buf);
  } else {
    E* sb = slab + buf * C::SLAB_SYM;
    nxt.store(sb, C::PS, tid);
    FM_SYNC();
    fm_readout_products<E, DH, QT, NACC, 0, C::PS, 0>(sb, xs, xrow, DH, 1, true, yb, acc, lr, lh);
  }
}

template <typename E, int DH, int QT, int NACC>
FM_DEVICE void fm_readout_sym(const E* FM_RESTRICT state, bool quad, const E* xs, const int* xrow,
                              const typename Mma<E>::frag (*yb)[TokCfg<E, DH, QT>::NKS],
                              E* slab, fm_f32x16 (*acc)[NACC], int tid) {
  typedef TokCfg<E, DH, QT> C;
  const int lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  int buf = 0;
  if (quad) {
    TileRegs<E, SymBlk<E, DH, QT, 0>::SAB * DH, DH> first;
    first.load(state, DH, tid);
    fm_readout_sym_block<E, DH, QT, NACC, 0>(state, first, xs, xrow, yb, slab, acc, tid, buf);
  } else {
    // `state` is the order-1 slab itself
    TileRegs<E, DH, DH> one;
    one.load(state, DH, tid);
    one.store(slab, C::PS, tid);
    FM_SYNC();
    fm_readout_products<E, DH, QT, NACC, 0, C::PS, 0>(slab, xs, xrow, DH, 1, true, yb, acc, lr, lh);
  }
  FM_SYNC();
}

// ------------------------------------------------------------------------------
// k_probe_mfma: one wavefront; A[i][k] = i + 1 (k = 0) else 0 ... chosen so that
// D[i][j] = (i + 1) * 100 + (j + 1) identifies which (row, col) every lane/register
// holds.  A[i][k] = {i + 1 at k = 0, 1 at k = 1};  B[k][j] = {100 at k = 0, j + 1 at k = 1}.
// ------------------------------------------------------------------------------
FM_GLOBAL void k_probe_mfma(float* out_f16, float* out_f32) {
  const int lane = FM_TID_X & 63, lr = lane & 31, lh = lane >> 5;
  fm_half8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) { a[i] = fm_half(0.f); b[i] = fm_half(0.f); }
  if (lh == 0) { a[0] = fm_half(float(lr + 1)); a[1] = fm_half(1.f); b[0] = fm_half(100.f); b[1] = fm_half(float(lr + 1)); }
  fm_f32x16 c = fm_zero16();
  c = fm_mfma_f16(a, b, c);
#pragma unroll
  for (int e = 0; e < 16; ++e) out_f16[lane * 16 + e] = c[e];
  // f32: k = 0 supplied by lanes 0..31, k = 1 by lanes 32..63
  const float af = lh == 0 ? float(lr + 1) : 1.f;
  const float bf = lh == 0 ? 100.f : float(lr + 1);
  fm_f32x16 c2 = fm_zero16();
  c2 = fm_mfma_f32(af, bf, c2);
#pragma unroll
  for (int e = 0; e < 16; ++e) out_f32[lane * 16 + e] = c2[e];
}

// ------------------------------------------------------------------------------
// k_probe_lds_tr: one wavefront; a 16 x 64 _Float16 tile holding 64 * row + col (all exact); lane l
// reads through fm_lds_tr4 at (row l % 16, column 4 * (l / 16)) and writes its four values.
// ------------------------------------------------------------------------------
FM_GLOBAL void k_probe_lds_tr(float* out) {
  FM_SHARED fm_half tile[16 * 64];
  const int l = FM_TID_X & 63;
  for (int i = l; i < 16 * 64; i += 64) tile[i] = fm_half(float(i));
  FM_SYNC();
  const fm_half4 v = fm_lds_tr4(tile + (l % 16) * 64 + 4 * (l / 16));
#pragma unroll
  for (int t = 0; t < 4; ++t) out[l * 4 + t] = float(v[t]);
}

