// Causal attention with more keys than queries (query i sees keys 0 .. nk - nq + i, the
// alignment of fastmax_cuda_forward.cu:161-172: the first nk - nq keys are summed before the
// first query).  The sums over keys split at nk - nq into a part every query sees (the head,
// an unmasked problem) and a square causal part (the tail); numerator and denominator add:
//   o = (o_head * g_head + o_tail * g_tail) / (g_head + g_tail),   g = g_head + g_tail.
// The backward needs no such step for dk and dv (the kernels take the final o and g, and
// the two parts write disjoint key ranges); dq is the sum of the two parts' dq.
#pragma once
#include "fm_kernels.h"

// o, g hold the tail's result on entry and the merged result on exit.  Eight features per thread;
// grid (ceil(n * DH / 8 / 256), bh).
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_merge_parts(TRef<const TIO> oa, TRef<const float> ga, TRef<TIO> o, TRef<float> g, int n) {
  constexpr int PER = DH / 8;
  const int bh = FM_BID_Y;
  const int64_t i = int64_t(FM_BID_X) * 256 + FM_TID_X;
  const int tok = int(i / PER), d0 = int(i % PER) * 8;
  if (tok >= n) return;
  const float wa = ga.base(bh)[int64_t(tok) * ga.s_n], wb = g.base(bh)[int64_t(tok) * g.s_n];
  const float inv = 1.0f / (wa + wb);
  float a[8], b[8];
  IO<TIO>::ld8(oa.base(bh) + int64_t(tok) * oa.s_n + d0, oa.vec != 0, a);
  IO<TIO>::ld8(o.base(bh) + int64_t(tok) * o.s_n + d0, o.vec != 0, b);
#pragma unroll
  for (int j = 0; j < 8; ++j) b[j] = (a[j] * wa + b[j] * wb) * inv;
  IO<TIO>::st8(o.base(bh) + int64_t(tok) * o.s_n + d0, o.vec != 0, b);
}

// g += ga, after every thread of k_merge_parts has read the old g (a launch of its own).
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_merge_denominators(TRef<const float> ga, TRef<float> g, int n) {
  const int bh = FM_BID_Y, tok = FM_BID_X * 256 + FM_TID_X;
  if (tok < n) g.base(bh)[int64_t(tok) * g.s_n] += ga.base(bh)[int64_t(tok) * ga.s_n];
}

// out += a, eight features per thread; grid (ceil(n * DH / 8 / 256), bh).
template <typename TIO, int DH>
FM_GLOBAL void FM_LAUNCH_BOUNDS(256) k_add_rows(TRef<const TIO> a, TRef<TIO> out, int n) {
  constexpr int PER = DH / 8;
  const int bh = FM_BID_Y;
  const int64_t i = int64_t(FM_BID_X) * 256 + FM_TID_X;
  const int tok = int(i / PER), d0 = int(i % PER) * 8;
  if (tok >= n) return;
  float x[8], y[8];
  IO<TIO>::ld8(a.base(bh) + int64_t(tok) * a.s_n + d0, a.vec != 0, x);
  IO<TIO>::ld8(out.base(bh) + int64_t(tok) * out.s_n + d0, out.vec != 0, y);
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] += x[j];
  IO<TIO>::st8(out.base(bh) + int64_t(tok) * out.s_n + d0, out.vec != 0, y);
}
