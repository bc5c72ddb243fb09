// Bench-only aids, compiled only into libfastmax_hip_bench.so (-DFM_BENCH_AIDS), never into the product
// library: two yardstick kernels for what the matrix cores sustain on a device, the per-kernel event timing
// of the launch paths, and the C declarations of their entry points.
#pragma once
#include "fm_kernels.h"

extern "C" {
/* Between begin and end the library brackets every kernel it launches with HIP events on the launch stream;
 * end waits for them and returns how many launches were recorded, filling up to `capacity` entries with the
 * kernel id (0 transpose, 1 backward prep, 2 state build, 3 forward, 4 dQ, 5 dK, 6 normalise, 7 dV, 8 dK and
 * dV in one pass) and its duration.  Process-global and not re-entrant. */
int fastmax_profile_begin(void);
int fastmax_profile_end(int* kernel_ids, float* milliseconds, int capacity);
/* `workgroups` workgroups of four wavefronts each issue `iters` rounds of eight independent 32x32x16 _Float16
 * matrix products on register operands: workgroups * 4 * iters * 8 * 32768 flop with no memory traffic; timed
 * by the caller with events on `hip_stream`.  out: workgroups * 256 floats (checksums). */
int fastmax_probe_mfma_rate(int workgroups, int iters, float* out, void* hip_stream);
/* The same with the operands coming out of LDS the way the dense kernels' do (see k_probe_mix):
 * workgroups * 4 * iters * 16 * own_tiles * 32768 flop.  own_tiles = 1 is built for two workgroups per CU, 2 for one. */
int fastmax_probe_mix_rate(int workgroups, int iters, int own_tiles, float* out, void* hip_stream);
}

// ------------------------------------------------------------------------------
// k_probe_mfma_rate: what the matrix cores sustain on this device with nothing in their way: every
// wavefront issues `iters` rounds of eight independent 32x32x16 _Float16 products on register
// operands (no memory, no LDS, no vector work).  2 * 32 * 32 * 16 flop per product.
// ------------------------------------------------------------------------------
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, 1) k_probe_mfma_rate(float* out, int iters) {
  fm_half8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) { a[i] = fm_half(float((FM_TID_X & 7) + i) * 0.125f); b[i] = fm_half(float(i) * 0.25f); }
  fm_f32x16 acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = fm_zero16();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = fm_mfma_f16(a, b, acc[i]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[i][e];
  out[FM_BID_X * FM_THREADS + FM_TID_X] = s;
}

// ------------------------------------------------------------------------------
// k_probe_mix: what the matrix cores sustain when their operands come out of LDS the way the dense kernels'
// do.  Per round and own tile a wavefront issues the 16 products of one 32x32 tile pair of the dK + dV pass;
// their streamed operands are 8 row fragments (16-byte LDS reads) and 8 transposed fragments (16 transposing
// 8-byte reads) per round, shared by the TILES own tiles of the wavefront, and 64 packed-half vector
// instructions per own tile stand for the polynomial.  No global memory, no barrier inside the loop.
// 2 * 32 * 32 * 16 flop per product.  TILES = 1 runs at two workgroups per CU like the dK + dV pass.
// ------------------------------------------------------------------------------
template <int TILES>
FM_GLOBAL void FM_LAUNCH_BOUNDS2(FM_THREADS, (TILES == 1 ? 2 : 1)) k_probe_mix(float* out, int iters) {
  typedef Mma<fm_half> M;
  typedef M::frag frag;
  constexpr int PQ = 64 + M::PAD;
  FM_SHARED fm_half tiles[4 * 32 * PQ];                  // two pairs of 32-token row tiles (x, y)
  const int tid = FM_TID_X, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  for (int i = tid; i < 4 * 32 * PQ; i += FM_THREADS) tiles[i] = fm_half(0.001f * float(i & 63));
  FM_SYNC();
  frag own[TILES][4];
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int i = 0; i < 8; ++i) own[t][ks][i] = fm_half(0.01f * float((lane + i + ks + t) & 15));
  fm_f32x16 acc[TILES][4];
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int a = 0; a < 4; ++a) acc[t][a] = fm_zero16();
  fm_half2 v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) { v[i][0] = fm_half(0.5f + float(i)); v[i][1] = fm_half(0.25f); }
  const fm_half2 c1 = {fm_half(1.0001f), fm_half(0.9999f)}, c2 = {fm_half(1e-4f), fm_half(-1e-4f)};
  for (int it = 0; it < iters; ++it) {
    const fm_half* X = tiles + (it & 1) * 2 * 32 * PQ;   // the two buffers in turn, as the stages alternate
    const fm_half* Y = X + 32 * PQ;
    frag xf[4], yf[4], xt[2][2], yt[2][2];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      xf[ks] = M::load(X + lr * PQ + ks * M::KSTEP + lh * M::KPL);
      yf[ks] = M::load(Y + lr * PQ + ks * M::KSTEP + lh * M::KPL);
    }
#pragma unroll
    for (int ss = 0; ss < 2; ++ss)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        xt[mt][ss] = M::load_tr(X, PQ, 16 * ss, 32 * mt, lane);
        yt[mt][ss] = M::load_tr(Y, PQ, 16 * ss, 32 * mt, lane);
      }
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        acc[t][0] = M::mma(xf[ks], own[t][ks], acc[t][0]);
        acc[t][1] = M::mma(yf[ks], own[t][ks], acc[t][1]);
      }
#pragma unroll
      for (int q = 0; q < 64; ++q) v[q & 7] = v[q & 7] * c1 + c2;
#pragma unroll
      for (int ss = 0; ss < 2; ++ss)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          acc[t][2] = M::mma(xt[mt][ss], own[t][ss], acc[t][2]);
          acc[t][3] = M::mma(yt[mt][ss], own[t][2 + ss], acc[t][3]);
        }
    }
  }
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int e = 0; e < 16; ++e) sum += acc[t][a][e];
#pragma unroll
  for (int i = 0; i < 8; ++i) sum += float(v[i][0]) + float(v[i][1]);
  out[FM_BID_X * FM_THREADS + tid] = sum;
}

