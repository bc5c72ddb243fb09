// Driver for the CPU build of the kernel sources (host simulator) under AddressSanitizer: a few shapes through the
// C ABI, forward and backward; the simulator keeps LDS and all tensors on the heap, so an index out of bounds in a
// kernel is reported.  Built and run by tests/test_hostsim.py when FASTMAX_HOSTSIM_ASAN=1.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <cmath>
#include "fastmax_hip.h"
static uint16_t bf16(float x) { uint32_t u; memcpy(&u, &x, 4); return uint16_t((u + 0x7fff + ((u >> 16) & 1)) >> 16); }
static float frand() { return float(rand()) / RAND_MAX * 2.f - 1.f; }
static int run(int bh, int n, int d, int p, int chunk, int dtype, int save) {
  FastmaxDesc D; memset(&D, 0, sizeof D);
  D.bh = bh; D.nq = D.nk = n; D.d = d; D.dtype = dtype; D.mask = 1; D.p = p; D.a0 = 1; D.a1 = 1; D.a2 = .5f;
  D.inv_tau = 1.f / (2.f * std::sqrt(float(d))); D.chunk = chunk; D.flags = save ? FASTMAX_FLAG_SAVE_FOR_BACKWARD : 0;
  FastmaxStrides s = {int64_t(n) * d, d, 0, 0};
  D.sq = D.sk = D.sv = D.so = D.sdo = D.sdq = D.sdk = D.sdv = s;
  D.sg.bh = n; D.sg.n = 1;
  size_t fb, bb; int st = fastmax_workspace_bytes(&D, &fb, &bb); if (st) return st;
  const size_t esz = dtype == FASTMAX_BF16 ? 2 : 4, ne = size_t(bh) * n * d;
  std::vector<char> q(ne * esz), k(ne * esz), v(ne * esz), go(ne * esz), o(ne * esz), dq(ne * esz), dk(ne * esz), dv(ne * esz);
  std::vector<float> g(size_t(bh) * n);
  for (size_t i = 0; i < ne; ++i)
    for (char* b : {q.data(), k.data(), v.data(), go.data()}) {
      const float x = frand();
      if (esz == 2) reinterpret_cast<uint16_t*>(b)[i] = bf16(x); else reinterpret_cast<float*>(b)[i] = x;
    }
  void* fws = aligned_alloc(256, (fb + 255) / 256 * 256); void* bws = aligned_alloc(256, (bb + 255) / 256 * 256);
  st = fastmax_forward(&D, q.data(), k.data(), v.data(), o.data(), g.data(), fws, fb, nullptr);
  if (!st) st = save ? fastmax_backward_saved(&D, q.data(), k.data(), v.data(), o.data(), g.data(), go.data(), dq.data(), dk.data(), dv.data(), fws, fb, bws, bb, nullptr)
                     : fastmax_backward(&D, q.data(), k.data(), v.data(), o.data(), g.data(), go.data(), dq.data(), dk.data(), dv.data(), bws, bb, nullptr);
  free(fws); free(bws);
  double sum = 0; for (float x : g) sum += x;
  printf("bh=%d n=%d d=%d p=%d chunk=%d dtype=%d save=%d -> status %d, sum g %.3f\n", bh, n, d, p, chunk, dtype, save, st, sum);
  return st;
}
// the two element-wise passes (key RPE, output noise) on a ragged shape, in place
static int run_pointwise(int bh, int n, int d, int dtype) {
  FastmaxNormDesc N{};
  N.bh = bh; N.n = n; N.d = d; N.dtype = dtype;
  N.sx.bh = int64_t(n) * d; N.sx.n = d; N.sy = N.sx;
  const size_t esz = dtype == FASTMAX_BF16 ? 2 : 4;
  std::vector<unsigned char> x(size_t(bh) * n * d * esz, 0), noise(x.size(), 0);
  std::vector<float> rpe(size_t(2 * n - 1) * d, 0.25f);
  int st = fastmax_key_rpe(&N, x.data(), rpe.data(), x.data(), 2.0f, nullptr);
  if (!st) st = fastmax_output_noise(&N, x.data(), noise.data(), x.data(), 0.5f, nullptr);
  printf("pointwise bh=%d n=%d d=%d dtype=%d -> status %d\n", bh, n, d, dtype, st);
  return st;
}
// the decoding state: a prompt absorbed, then single-token steps (buffers of exactly the sizes the library names)
static int run_decode(int bh, int d, int p, int prompt, int steps, int dtype) {
  FastmaxDesc D; memset(&D, 0, sizeof D);
  D.bh = bh; D.nq = 1; D.nk = prompt; D.d = d; D.dtype = dtype; D.mask = 1; D.p = p; D.a0 = 1; D.a1 = 1; D.a2 = .5f;
  D.inv_tau = 1.f / (2.f * std::sqrt(float(d)));
  FastmaxStrides s = {int64_t(prompt) * d, d, 0, 0}, s1 = {int64_t(d), d, 0, 0};
  D.sq = s1; D.sk = D.sv = s; D.so = s1; D.sg.bh = 1; D.sg.n = 1;
  const size_t esz = dtype == FASTMAX_BF16 ? 2 : 4, ne = size_t(bh) * prompt * d;
  std::vector<char> k(ne * esz), v(ne * esz), q1(size_t(bh) * d * esz), k1(q1.size()), v1(q1.size()), o1(q1.size());
  auto fill = [&](std::vector<char>& b) {
    for (size_t i = 0; i < b.size() / esz; ++i) {
      const float x = frand();
      if (esz == 2) reinterpret_cast<uint16_t*>(b.data())[i] = bf16(x); else reinterpret_cast<float*>(b.data())[i] = x;
    }
  };
  fill(k); fill(v); fill(q1); fill(k1); fill(v1);
  const size_t sb = fastmax_decode_state_bytes(&D), cb = fastmax_decode_scratch_bytes(&D);
  if (!sb || !cb) return 99;
  float* state = static_cast<float*>(aligned_alloc(256, (sb + 255) / 256 * 256));
  memset(state, 0, sb);
  float* scratch = static_cast<float*>(aligned_alloc(256, (cb + 255) / 256 * 256));
  std::vector<float> g(bh);
  int st = fastmax_decode_absorb(&D, k.data(), v.data(), state, nullptr);
  D.sk = D.sv = s1;
  for (int i = 0; i < steps && !st; ++i)
    st = fastmax_decode_step(&D, q1.data(), k1.data(), v1.data(), state, o1.data(), g.data(), scratch, nullptr);
  free(state); free(scratch);
  printf("decode bh=%d d=%d p=%d prompt=%d steps=%d dtype=%d -> status %d, g[0] %.3f\n", bh, d, p, prompt, steps, dtype, st, g[0]);
  return st;
}
int main() {
  int bad = 0;
  bad |= run_pointwise(3, 333, 64, FASTMAX_BF16);
  bad |= run_pointwise(2, 70, 32, FASTMAX_F32);
  bad |= run_decode(2, 64, 2, 37, 2, FASTMAX_BF16);
  bad |= run_decode(3, 32, 1, 5, 2, FASTMAX_F32);
  bad |= run_decode(1, 64, 2, 150, 1, FASTMAX_BF16);  // a prompt summed with matrix instructions (two tiles, the second ragged)
  bad |= run(1, 300, 64, 2, 256, FASTMAX_BF16, 1);    // order-2 walk held per value column (two segments), saved and rebuilt
  bad |= run(1, 300, 64, 2, 256, FASTMAX_BF16, 0);
  bad |= run(1, 600, 32, 2, 256, FASTMAX_BF16, 1);    // order-2 walk (a CU to itself: two buffers), both walks
  bad |= run(1, 600, 32, 2, 256, FASTMAX_BF16, 0);
  bad |= run(1, 520, 64, 2, 256, FASTMAX_BF16, 1);
  bad |= run(1, 1100, 32, 1, 0, FASTMAX_BF16, 1);     // order-1 runs of segments
  bad |= run(3, 1300, 64, 1, 0, FASTMAX_BF16, 0);
  bad |= run(2, 200, 64, 2, 0, FASTMAX_BF16, 1);      // one segment, dense kernels
  bad |= run(1, 200, 128, 2, 0, FASTMAX_BF16, 1);     // heads of 128: four accumulator tiles per feature axis
  bad |= run(1, 150, 128, 1, 0, FASTMAX_BF16, 0);
  bad |= run(1, 300, 32, 2, 256, FASTMAX_F32, 1);
  return bad;
}
