// Thin portability layer between the kernels and what runs them.
//
// The kernels are written once against the names below.  The normal build is
// hipcc for gfx950.  A second, test-only build (-DFM_HOSTSIM, plain C++) maps
// the same names onto a host-thread simulator so that indexing and lane layouts
// can be checked without a GPU; the shipped library never defines FM_HOSTSIM.
#pragma once
#include <cstddef>
#include <cstdint>

typedef _Float16 fm_half;
typedef _Float16 fm_half2 __attribute__((ext_vector_type(2)));
typedef _Float16 fm_half4 __attribute__((ext_vector_type(4)));
typedef _Float16 fm_half8 __attribute__((ext_vector_type(8)));
typedef float fm_f32x2 __attribute__((ext_vector_type(2)));
typedef float fm_f32x4 __attribute__((ext_vector_type(4)));
typedef float fm_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t fm_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t fm_u32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t fm_bf16;  // raw storage of a bfloat16

#if defined(FM_HOSTSIM)
// ------------------------------------------------------------------ host simulator
#include <cmath>
#include "hostsim.h"
#define FM_GLOBAL
#define FM_DEVICE inline
#define FM_ALWAYS_INLINE __attribute__((always_inline))
#define FM_HOST_DEVICE
#define FM_LAUNCH_BOUNDS(n)
#define FM_LAUNCH_BOUNDS2(n, m)
#define FM_RESTRICT
#define FM_UNIFORM(x) (x)
#define FM_OPAQUE_ZERO() 0
#define FM_SCHED_FENCE()
#define FM_SCHED_MFMA_DS(n)
#define FM_KEEP_BRANCH()
#define FM_WAIT_GLOBAL_LOADS()
typedef void* fm_stream_t;
typedef hostsim::Dim3 fm_dim3;
#define FM_TID_X (int(hostsim::g_t.tid.x))
#define FM_BID_X (int(hostsim::g_t.bid.x))
#define FM_BID_Y (int(hostsim::g_t.bid.y))
#define FM_BID_Z (int(hostsim::g_t.bid.z))
#define FM_GDIM_X (int(hostsim::g_t.gdim.x))
#define FM_GDIM_Y (int(hostsim::g_t.gdim.y))
#define FM_GDIM_Z (int(hostsim::g_t.gdim.z))
#define FM_SYNC() hostsim::syncthreads()
#define FM_WAVE_SYNC() hostsim::syncthreads()
#define FM_DYN_SMEM(name) unsigned char* name = hostsim::g_t.blk->dyn_smem
#define FM_KERNEL_LAUNCH(kern, grid, block, smem, stream, ...) \
  hostsim::launch((grid), (block), (smem), [=]() { kern(__VA_ARGS__); })
inline int fm_after_launch() { return 0; }

FM_DEVICE fm_f32x16 fm_mfma_f16(fm_half8 a, fm_half8 b, fm_f32x16 c) {
  fm_half av[8], bv[8]; float cv[16];
  for (int i = 0; i < 8; ++i) { av[i] = a[i]; bv[i] = b[i]; }
  for (int i = 0; i < 16; ++i) cv[i] = c[i];
  hostsim::mfma_32x32<fm_half, 8>(av, bv, cv);
  for (int i = 0; i < 16; ++i) c[i] = cv[i];
  return c;
}
FM_DEVICE fm_f32x16 fm_mfma_f32(float a, float b, fm_f32x16 c) {
  float cv[16];
  for (int i = 0; i < 16; ++i) cv[i] = c[i];
  hostsim::mfma_32x32<float, 1>(&a, &b, cv);
  for (int i = 0; i < 16; ++i) c[i] = cv[i];
  return c;
}
FM_DEVICE float fm_shfl_xor(float v, int m) { return hostsim::shfl(v, hostsim::g_t.lane ^ m); }
FM_DEVICE int fm_shfl_xor_i(int v, int m) { return hostsim::shfl(v, hostsim::g_t.lane ^ m); }
FM_DEVICE float fm_dot2(fm_half2 a, fm_half2 b, float c) { return float(a[0]) * float(b[0]) + float(a[1]) * float(b[1]) + c; }
// Transposing LDS read (ds_read_b64_tr_b16): every lane names four consecutive halves; inside each
// group of 16 lanes, lane i receives element i % 4 of the words named by lanes i/4, 4 + i/4,
// 8 + i/4 and 12 + i/4 (layout read off the instruction on an MI355X by a probe kernel).
FM_DEVICE fm_half4 fm_lds_tr4(const fm_half* p) {
  fm_half4 w;
  __builtin_memcpy(&w, p, 8);
  const int lane = hostsim::g_t.lane, g = lane & ~15, i = lane & 15;
  fm_half4 r;
  for (int t = 0; t < 4; ++t) {
    const fm_half4 o = hostsim::shfl(w, g + 4 * t + i / 4);
    r[t] = o[i % 4];
  }
  return r;
}
FM_DEVICE float fm_fmaxf(float a, float b) { return a != a ? b : (b != b ? a : (a > b ? a : b)); }   // drops a NaN, like fmaxf
FM_DEVICE float fm_clampf(float x, float lim) { return x > lim ? lim : (x < -lim ? -lim : x); }
FM_DEVICE float fm_rsqrtf(float a) { return 1.0f / std::sqrt(a); }
FM_DEVICE float fm_sqrtf(float a) { return std::sqrt(a); }

#else
// ------------------------------------------------------------------ gfx950
#include <hip/hip_runtime.h>
#define FM_GLOBAL __global__
#define FM_DEVICE __device__ __forceinline__
#define FM_ALWAYS_INLINE __attribute__((always_inline))
#define FM_HOST_DEVICE __host__ __device__
#define FM_LAUNCH_BOUNDS(n) __launch_bounds__(n)
#define FM_LAUNCH_BOUNDS2(n, m) __launch_bounds__(n, m)
#define FM_RESTRICT __restrict__
// a value that is the same in every lane of the wavefront, moved to a scalar register so that
// branches on it are scalar branches
#define FM_UNIFORM(x) __builtin_amdgcn_readfirstlane(x)
// A zero the optimiser cannot see through: added to an LDS offset it keeps two reads of the
// same tile apart, so the second is a fresh read instead of 16 more live registers.
static __device__ __forceinline__ int fm_opaque_zero() { int z = 0; asm volatile("" : "+v"(z)); return z; }
#define FM_OPAQUE_ZERO() fm_opaque_zero()
// Nothing is scheduled across this point (keeps the live ranges of one phase out of the next).
#define FM_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
// Asks the instruction scheduler to interleave the LDS reads of this block with its matrix
// instructions (strategy 0: small products, 1: one wavefront's view); it changes the order of
// instructions only.  On MI355X the dense stages run 1 to 2 % faster with it.
#define FM_SCHED_MFMA_DS(n) __builtin_amdgcn_iglp_opt(n)
// Inside a rarely taken wavefront-uniform branch: keeps it a branch (the optimiser would
// otherwise run its body on every pass and select the result).
#define FM_KEEP_BRANCH() asm volatile("")
// Waits for every global load of the wavefront that is still in flight (s_waitcnt vmcnt(0), the other counters left
// alone).  Ahead of a software-pipelined loop it tells the compiler that nothing is pending on entry, so the loop
// head does not inherit a full wait from the prologue's loads on every iteration.
#define FM_WAIT_GLOBAL_LOADS() __builtin_amdgcn_s_waitcnt(0x0F70)
typedef hipStream_t fm_stream_t;
typedef dim3 fm_dim3;
#define FM_TID_X (int(threadIdx.x))
#define FM_BID_X (int(blockIdx.x))
#define FM_BID_Y (int(blockIdx.y))
#define FM_BID_Z (int(blockIdx.z))
#define FM_GDIM_X (int(gridDim.x))
#define FM_GDIM_Y (int(gridDim.y))
#define FM_GDIM_Z (int(gridDim.z))
#define FM_SYNC() __syncthreads()
// Between LDS writes and reads of the same wavefront (lanes exchange data through a region no other wavefront touches):
// the LDS serves a wavefront's operations in order, so only the compiler has to keep them in order.
#define FM_WAVE_SYNC() do { __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront"); } while (0)
#define FM_DYN_SMEM(name) extern __shared__ __align__(16) unsigned char name[]
// A launch the runtime refuses leaves its error as the calling thread's last error.  Only an error that
// appears across the launch is this library's: it is taken (cleared) and remembered until
// fm_after_launch() asks; an error some other library left pending before the launch stays where its
// owner will look for it and is not blamed on the launch.
inline thread_local int fm_launch_refused = 0;
#define FM_KERNEL_LAUNCH(kern, grid, block, smem, stream, ...)                                      \
  do {                                                                                              \
    const bool fm_clean_ = hipPeekAtLastError() == hipSuccess;                                      \
    hipLaunchKernelGGL(kern, (grid), (block), (smem), (stream), __VA_ARGS__);                       \
    if (fm_clean_ && hipPeekAtLastError() != hipSuccess) { (void)hipGetLastError(); fm_launch_refused = 1; } \
  } while (0)
// 0, or non-zero when a launch since the last call was refused
inline int fm_after_launch() { const int r = fm_launch_refused; fm_launch_refused = 0; return r; }

FM_DEVICE fm_f32x16 fm_mfma_f16(fm_half8 a, fm_half8 b, fm_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
FM_DEVICE fm_f32x16 fm_mfma_f32(float a, float b, fm_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
FM_DEVICE float fm_shfl_xor(float v, int m) { return __shfl_xor(v, m, 64); }
FM_DEVICE int fm_shfl_xor_i(int v, int m) { return __shfl_xor(v, m, 64); }
FM_DEVICE float fm_dot2(fm_half2 a, fm_half2 b, float c) { return __builtin_amdgcn_fdot2(a, b, c, false); }
// Transposing LDS read (ds_read_b64_tr_b16): every lane names four consecutive halves; inside each
// group of 16 lanes, lane i receives element i % 4 of the words named by lanes i/4, 4 + i/4,
// 8 + i/4 and 12 + i/4 (layout read off the instruction on an MI355X by a probe kernel).
FM_DEVICE fm_half4 fm_lds_tr4(const fm_half* p) {
  typedef short fm_s16x4 __attribute__((ext_vector_type(4)));
  const fm_s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) fm_s16x4*)(p));
  fm_half4 r;
  __builtin_memcpy(&r, &v, 8);
  return r;
}
FM_DEVICE float fm_fmaxf(float a, float b) { return fmaxf(a, b); }
// clamp to [-lim, lim] in one instruction (v_med3_f32)
FM_DEVICE float fm_clampf(float x, float lim) { return __builtin_amdgcn_fmed3f(x, -lim, lim); }
FM_DEVICE float fm_rsqrtf(float a) { return rsqrtf(a); }
FM_DEVICE float fm_sqrtf(float a) { return sqrtf(a); }
#endif

// ---- bf16 <-> f32 (round to nearest even), usable on both builds -------------
FM_DEVICE float fm_bf16_to_f32(fm_bf16 v) {
  uint32_t u = uint32_t(v) << 16;
  float f;
  __builtin_memcpy(&f, &u, 4);
  return f;
}
FM_DEVICE fm_bf16 fm_f32_to_bf16(float f) {
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return fm_bf16((u >> 16) | 0x40u);  // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return fm_bf16(u >> 16);
}
