// Host-side functional simulator for the HIP kernels of this repository.
//
// TEST INFRASTRUCTURE ONLY.  The kernel sources are compiled a second time as
// plain C++ (clang++ -x c++ -DFM_HOSTSIM) against this header so that their
// indexing, lane layouts and bounds can be exercised on a machine without a
// GPU, under AddressSanitizer.  Every workgroup is run by real OS threads (one
// per work-item), workgroups run one after another, `__syncthreads` is a
// barrier over the workgroup, and the wave-wide matrix instructions are
// emulated by exchanging the operands of the 64 lanes of a wave through a
// per-wave scratch area.  Nothing in the shipped library includes this file.
#pragma once
#include <condition_variable>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

namespace hostsim {

struct Dim3 { unsigned x = 1, y = 1, z = 1; Dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {} };

class Barrier {
 public:
  void reset(int n) { n_ = n; count_ = 0; gen_ = 0; }
  void wait() {
    std::unique_lock<std::mutex> lk(m_);
    int g = gen_;
    if (++count_ == n_) { count_ = 0; ++gen_; cv_.notify_all(); }
    else cv_.wait(lk, [&] { return gen_ != g; });
  }
 private:
  std::mutex m_; std::condition_variable cv_; int n_ = 1, count_ = 0, gen_ = 0;
};

struct WaveCtx {
  Barrier bar;
  alignas(64) unsigned char a[64][64];   // per-lane operand A (up to 64 bytes)
  alignas(64) unsigned char b[64][64];   // per-lane operand B
};

struct BlockCtx {
  Barrier bar;
  std::vector<WaveCtx> waves;
  unsigned char* dyn_smem = nullptr;
};

struct ThreadCtx {
  Dim3 tid, bid, bdim, gdim;
  BlockCtx* blk = nullptr;
  WaveCtx* wave = nullptr;
  int lane = 0;
};

inline thread_local ThreadCtx g_t;

template <class F>
void launch(Dim3 grid, Dim3 block, size_t dyn_smem_bytes, F&& body) {
  const int nthreads = int(block.x * block.y * block.z);
  if (nthreads % 64 != 0) { std::fprintf(stderr, "hostsim: block size must be a multiple of 64\n"); std::abort(); }
  BlockCtx blk;
  blk.waves = std::vector<WaveCtx>(nthreads / 64);
  
  for (unsigned bz = 0; bz < grid.z; ++bz)
    for (unsigned by = 0; by < grid.y; ++by)
      for (unsigned bx = 0; bx < grid.x; ++bx) {
        blk.bar.reset(nthreads);
        for (auto& w : blk.waves) w.bar.reset(64);
        // exact-size allocation so that AddressSanitizer sees overruns of the dynamic LDS
        unsigned char* dyn = static_cast<unsigned char*>(std::malloc(dyn_smem_bytes ? dyn_smem_bytes : 1));
        blk.dyn_smem = dyn;
        std::vector<std::thread> ths;
        ths.reserve(nthreads);
        for (int t = 0; t < nthreads; ++t) {
          ths.emplace_back([&, t] {
            g_t.tid = Dim3(t % block.x, (t / block.x) % block.y, t / (block.x * block.y));
            g_t.bid = Dim3(bx, by, bz);
            g_t.bdim = block; g_t.gdim = grid;
            g_t.blk = &blk; g_t.wave = &blk.waves[t / 64]; g_t.lane = t % 64;
            body();
          });
        }
        for (auto& th : ths) th.join();
        std::free(dyn);
      }
}

inline void syncthreads() { g_t.blk->bar.wait(); }

// ---- wave-level data exchange ------------------------------------------------
template <class T>
inline T shfl(T v, int src_lane) {
  static_assert(sizeof(T) <= 64, "operand too large");
  WaveCtx* w = g_t.wave;
  std::memcpy(w->a[g_t.lane], &v, sizeof(T));
  w->bar.wait();
  T r; std::memcpy(&r, w->a[src_lane & 63], sizeof(T));
  w->bar.wait();
  return r;
}

// D(32x32) += A(32xK) * B(Kx32), K = 2*KPL.  Lane l supplies A[row l%32][k] and
// B[k][col l%32] for k = (l/32)*KPL .. +KPL-1, and owns D[8*(e/4)+4*(l/32)+e%4][l%32].
template <class E, int KPL>
inline void mfma_32x32(const E* a, const E* b, float* acc) {
  WaveCtx* w = g_t.wave;
  const int lane = g_t.lane;
  std::memcpy(w->a[lane], a, sizeof(E) * KPL);
  std::memcpy(w->b[lane], b, sizeof(E) * KPL);
  w->bar.wait();
  const int col = lane & 31, half = lane >> 5;
  for (int e = 0; e < 16; ++e) {
    const int row = 8 * (e / 4) + 4 * half + (e % 4);
    float s = 0.f;
    for (int k = 0; k < 2 * KPL; ++k) {
      E av, bv;
      std::memcpy(&av, w->a[row + 32 * (k / KPL)] + sizeof(E) * (k % KPL), sizeof(E));
      std::memcpy(&bv, w->b[col + 32 * (k / KPL)] + sizeof(E) * (k % KPL), sizeof(E));
      s += float(av) * float(bv);
    }
    acc[e] += s;
  }
  w->bar.wait();
}

}  // namespace hostsim
