// C ABI of libfastmax_hip.so: argument validation, workspace planning and the
// launch sequences.  See include/fastmax_hip.h for the contract of each entry.
#include "fastmax_hip.h"
#include "fm_kernels.h"
#include "fm_tok.h"
#include "fm_norm.h"
#include "fm_split.h"
#include "fm_decode.h"
#include "fm_o1.h"
#include "fm_pointwise.h"
#include "fm_walk_sym.h"
#if defined(FM_BENCH_AIDS)
#include "fm_bench_aids.h"
#endif
// the one head size beyond 64: served by the _Float16 token kernels on dense tiles (see validate)
static constexpr int FM_WIDE_HEAD = 128;
#include <atomic>
#include <cmath>
#include <mutex>
#include <unordered_map>
#include <vector>

// ---- static scratch of fastmax_forward_static ------------------------------------------------
// Device memory that belongs to the loaded library: every GPU the library runs on holds its own copy
// of this array, at its own address, until the process ends.
#if defined(FM_HOSTSIM)
alignas(256) static unsigned char scratch[FASTMAX_STATIC_SCRATCH_BYTES];
static inline int fm_static_scratch(void** out) { *out = scratch; return FASTMAX_OK; }
#else
static __device__ __align__(256) unsigned char scratch[FASTMAX_STATIC_SCRATCH_BYTES];
// In host code the array's name is only a handle for the runtime, not a device address.  The address
// on the current device is asked for once per device (with that device current) and kept; kernels and
// copies are only ever given that address.
static inline int fm_static_scratch(void** out) {
  enum { MAX_DEVICES = 64 };
  static std::mutex mu;
  static void* addr[MAX_DEVICES] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return FASTMAX_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(mu);
  if (!addr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return FASTMAX_ERR_LAUNCH;
    addr[dev] = ptr;
  }
  *out = addr[dev];
  return FASTMAX_OK;
}
#endif

namespace {

inline int fm_launch_status() { return fm_after_launch() ? FASTMAX_ERR_LAUNCH : FASTMAX_OK; }
#if defined(FM_HOSTSIM)
inline void fm_allow_lds(const void*, size_t) {}
#else
// Dynamic LDS above the 64 KiB default has to be allowed once per kernel function (and device); the
// attribute call costs microseconds of host time, so it is made the first time a kernel asks for more
// than it has been granted so far and skipped afterwards.
inline void fm_allow_lds(const void* fn, size_t bytes) {
  if (bytes <= 64 * 1024) return;
  struct Key { const void* fn; int dev; bool operator==(const Key& o) const { return fn == o.fn && dev == o.dev; } };
  struct Hash { size_t operator()(const Key& k) const { return std::hash<const void*>()(k.fn) ^ (size_t(k.dev) * 0x9e3779b97f4a7c15ull); } };
  static std::mutex mu;
  static std::unordered_map<Key, size_t, Hash> granted;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  std::lock_guard<std::mutex> lock(mu);
  size_t& have = granted[Key{fn, dev}];
  if (bytes <= have) return;
  if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes)) == hipSuccess) have = bytes;
}
#endif

// ---- per-kernel timing: compiled only into the bench build of this file (-DFM_BENCH_AIDS); in the product
// library a ProfScope is an empty object and no launch touches any process-wide state ---------------------
enum { FM_K_TRANSPOSE = 0, FM_K_PREP_BWD = 1, FM_K_BUILD = 2, FM_K_FWD = 3, FM_K_DQ = 4, FM_K_DK = 5, FM_K_NORM = 6, FM_K_DV = 7, FM_K_DKV = 8 };
#if defined(FM_HOSTSIM) || !defined(FM_BENCH_AIDS)
struct ProfScope { ProfScope(int, fm_stream_t) {} };
#else
struct ProfRec { int id; hipEvent_t a, b; };
std::atomic<bool> g_prof_on{false};   // read by every launch: atomic, so that a launch on another thread sees a whole value
std::vector<ProfRec> g_prof;
struct ProfScope {
  bool on; fm_stream_t s; size_t idx;
  ProfScope(int id, fm_stream_t stream) : on(g_prof_on.load(std::memory_order_relaxed)), s(stream), idx(0) {
    if (!on) return;
    ProfRec r; r.id = id;
    hipEventCreate(&r.a); hipEventCreate(&r.b);
    hipEventRecord(r.a, s);
    g_prof.push_back(r); idx = g_prof.size() - 1;
  }
  ~ProfScope() { if (on) hipEventRecord(g_prof[idx].b, s); }
};
#endif

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
inline size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

struct Plan {
  bool half;            // compute type: _Float16 (bf16 interface) or float
  int esz;              // sizeof compute element
  int L, nseg, nslots;
  bool use_state, quad;
  bool rows_build;      // order-1 segment sums read the row-major copies: no transposed copy is written
  int o1_run;           // order-1 path: segments per run (see k_o1_sums)
  bool o1;              // order 1, causal, _Float16, 128-token segments: the path of fm_o1.h (reads the caller's tensors, no copies)
  bool qf;              // dense _Float16 kernels evaluate the order-2 weights in completed-square form (see TileMath)
  int npad_q, npad_k;
  float a0, a1, a2;     // polynomial on the score s = (q.k) / tau
  float sc;             // sqrt(1/tau), folded into q and k when they are converted
  // workspace offsets (bytes)
  size_t kt, vt, kr, vr, big, big2, small, run, runh, ores, fwd_bytes;
  bool keep_resid;      // the forward leaves o - bf16(o) for the backward (see TokArgs::out_resid)
  bool sym;             // order-2 states are built by the walk per value column (k_walk_sym): one layout, no transposed copy   // run, runh: see k_o1_sums
  bool save;
  size_t b_kr, b_vr, b_qr, b_kt, b_vt, b_qt, b_qct, b_gh, b_ght, b_cv, b_bigq, b_smallq, b_bigk, b_smallk, b_bigv, b_gpart, b_bq, b_bk, b_runq, b_runqh, b_runk, b_runkh, bwd_bytes;
};

bool strides_ok(const FastmaxStrides& s, int bh, int n, int d) {
  if (s.n < d && n > 1) return false;
  if (s.heads > 1) {                                   // batch and head strides
    if (bh % s.heads != 0) return false;
    if (s.bh <= 0) return false;
    if (s.b <= 0 && bh > s.heads) return false;
  } else if (s.bh <= 0 && bh > 1) {
    return false;
  }
  return s.n > 0 || n <= 1;
}

int validate(const FastmaxDesc* d) {
  if (!d) return FASTMAX_ERR_NULL;
  if (d->dtype != FASTMAX_F32 && d->dtype != FASTMAX_BF16) return FASTMAX_ERR_DTYPE;
  if (d->bh <= 0 || d->nq <= 0 || d->nk <= 0 || d->d <= 0) return FASTMAX_ERR_SHAPE;
  if (d->bh > 65535) return FASTMAX_ERR_SHAPE;
  // padded lengths, segment lengths and their byte counts are formed in 32- and 64-bit arithmetic that
  // assumes token counts and the segment length stay below 2^30
  if (d->nq > (1 << 30) || d->nk > (1 << 30) || d->chunk > (1 << 30)) return FASTMAX_ERR_SHAPE;
  if (d->p != 1 && d->p != 2) return FASTMAX_ERR_UNSUPPORTED;
  if (d->d != 32 && d->d != 64 && d->d != FM_WIDE_HEAD) return FASTMAX_ERR_UNSUPPORTED;
  if (d->d == FM_WIDE_HEAD) {
    // heads of 128: bf16 tensors on the _Float16 kernels, dense tiles only (no moment states, no normalisation fold,
    // no causal nk > nq): at that width the moment form only pays beyond about D^2 = 16 384 keys
    if (d->dtype != FASTMAX_BF16 || (d->flags & FASTMAX_FLAG_F32_COMPUTE) || !(d->a0 > 0.0f)) return FASTMAX_ERR_UNSUPPORTED;
    if (d->norm.q_keys || d->norm.k_keys || (d->mask && d->nk > d->nq)) return FASTMAX_ERR_UNSUPPORTED;
    if (d->flags & FASTMAX_FLAG_FORCE_MOMENTS) return FASTMAX_ERR_UNSUPPORTED;
  }
  if (d->mask && d->nq > d->nk) return FASTMAX_ERR_UNSUPPORTED;   // nk > nq: see SplitPlan
  if (d->chunk < 0) return FASTMAX_ERR_SHAPE;
  if (!(d->inv_tau > 0.0f) || !(d->inv_tau < 3.0e38f)) return FASTMAX_ERR_SHAPE;   // also rejects NaN
  if (d->norm.q_keys || d->norm.k_keys) {
    if (d->mask && d->nk > d->nq) return FASTMAX_ERR_UNSUPPORTED;                    // two parts would share one Jacobian
    if (!(d->norm.lim > 0.0f) || !(d->norm.lim < 3.0e38f)) return FASTMAX_ERR_SHAPE;
    if ((reinterpret_cast<uintptr_t>(d->norm.q_keys) | reinterpret_cast<uintptr_t>(d->norm.k_keys)) % 8) return FASTMAX_ERR_SHAPE;
  }
  return FASTMAX_OK;
}

// bytes of one `big` state array: the slots of all segments of all batch*heads and, when a slot is the
// order-1 slab alone, the padding that the readers' four-slab fetches may touch behind the last one
template <int DH> size_t big_array_bytes(int esz, bool quad, size_t slots) {
  if (!slots) return 0;
  return (slots * size_t(StateDims<DH>::stride(quad)) + (quad ? 0 : size_t(StateDims<DH>::PAD_SLABS) * StateDims<DH>::SLAB)) * esz;
}

int make_plan(const FastmaxDesc* d, Plan& p) {
  int st = validate(d);
  if (st != FASTMAX_OK) return st;
  // _Float16 arithmetic serves weights that are positive sums: with a0 <= 0 the weights f(s) change sign
  // around s = 0, numerator and denominator cancel, and 11 bits per weight no longer bound the error of
  // their ratio; such problems are computed in fp32 like the ones that ask for it
  p.half = d->dtype == FASTMAX_BF16 && !(d->flags & FASTMAX_FLAG_F32_COMPUTE) && d->a0 > 0.0f;
  p.esz = p.half ? 2 : 4;
  p.npad_q = int(round_up(d->nq, 256));
  p.npad_k = int(round_up(d->nk, 256));
  p.quad = d->p == 2 && d->a2 != 0.0f;
  p.a0 = d->a0;
  p.a1 = d->a1;
  p.a2 = p.quad ? d->a2 : 0.0f;
  p.sc = std::sqrt(std::fabs(d->inv_tau));
  const bool force_dense = (d->flags & FASTMAX_FLAG_FORCE_DENSE) != 0 || d->d == FM_WIDE_HEAD;
  if (d->mask) {
    // Segment length.  Dense tiles cost grows with L, the moment states cost the same per token
    // whatever L is (readout) plus the walk that builds them.  Measured on MI355X (D = 64, bf16):
    // order 2: one segment (no states at all) wins up to about 6000 tokens, 1024-token segments
    // beyond; order 1 (one D x D state per segment): one segment up to 1024 tokens (0.150 against 0.159 ms
    // per step at B*H = 128; at 1536 tokens, B*H = 96: 0.209 against 0.190),
    // 256-token segments beyond.
    // Order 1 on _Float16: 128-token segments, so that the backward of a segment is one workgroup's work (k_o1_bwd).
    const int auto_L = p.quad ? (d->nq > 6144 ? 1024 : p.npad_q) : (d->nq > 1024 ? (p.half ? 128 : 256) : p.npad_q);
    int L = d->chunk > 0 ? (d->chunk >= d->nq ? p.npad_q : int(round_up(d->chunk, 256))) : auto_L;
    if (force_dense || L > p.npad_q) L = p.npad_q;
    p.L = L;
    p.nseg = (d->nq + L - 1) / L;
    p.use_state = p.nseg > 1;
    p.nslots = p.use_state ? p.nseg : 0;
  } else {
    p.L = p.npad_k;
    p.nseg = 1;
    const bool force_m = (d->flags & FASTMAX_FLAG_FORCE_MOMENTS) != 0;
    p.use_state = force_m || (!force_dense && int64_t(d->nk) > int64_t(d->d) * d->d + d->d);
    p.nslots = p.use_state ? 1 : 0;
  }
  p.o1 = p.half && p.use_state && !p.quad && d->mask && p.L == FM_O1_SEG && d->nq == d->nk;
  p.rows_build = p.half && p.use_state && !p.quad && d->mask;
  {
    // f = (h^2 + kc) / (4 a2) with h = 2 a2 s + a1: worth it, and safe in _Float16, when a2 and kc are of ordinary size
    const float kc = 4.0f * p.a0 * p.a2 - p.a1 * p.a1;
    p.qf = p.half && p.quad && !p.use_state && std::fabs(p.a2) >= 0.0625f && std::fabs(p.a2) <= 4.0f &&
           std::fabs(kc) <= 1024.0f && std::fabs(p.a1) <= 64.0f && d->d <= 64;
  }
  {
    // _Float16, D = 64, and enough batch*heads that one walk per (four values, batch*head) fills the chip; smaller
    // problems sum their segments apart (k_build with seg_parallel)
    const int nsteps = d->mask ? p.nseg - 1 : 1;
    p.sym = p.half && d->d == 64 && p.quad && p.use_state && !(nsteps > 1 && d->bh * 16 < 256);
  }
  const size_t slots = size_t(d->bh) * p.nslots;
  const size_t bigarr = d->d == 64 ? big_array_bytes<64>(p.esz, p.quad, slots) : big_array_bytes<32>(p.esz, p.quad, slots);
  // fp32 part of a slot: Z and the two vector sums; the order-1 path of fm_o1.h keeps the two vectors only
  const size_t smallsz = p.o1 ? size_t(2) * d->d * 4 : size_t(d->d == 64 ? StateDims<64>::SMALL : StateDims<32>::SMALL) * 4;
  const size_t tq = p.o1 ? 0 : size_t(d->bh) * d->d * p.npad_q * p.esz;
  const size_t tk = p.o1 ? 0 : size_t(d->bh) * d->d * p.npad_k * p.esz;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align256(off + bytes); return o; };
  // transposed copies: only the order-2 state walk, the one-total order-1 walk and the fp32 kernels read them
  const bool need_t = !(p.half && (!p.use_state || p.rows_build));
  const size_t tkt = need_t ? tk : 0, tqt = need_t ? tq : 0;
  p.kt = take(tkt);
  p.vt = take(tkt);
  p.kr = take(tk);
  p.big = take(bigarr);
  p.small = take(size_t(d->bh) * p.nslots * smallsz);
  p.save = (d->flags & FASTMAX_FLAG_SAVE_FOR_BACKWARD) != 0;
  p.vr = take(p.save || p.half ? tk : 0);      // _Float16: the forward stages v rows (transposing LDS reads)
  p.big2 = take(p.save && !p.o1 && !p.sym ? bigarr : 0);
  // the order-1 path sums runs of segments: per batch*head and run one fp32 total and its compute-type slab
  p.o1_run = fm_o1_run_len(p.nseg, d->bh);
  const size_t nruns = p.o1 ? size_t(fm_o1_runs(p.nseg, p.o1_run)) : 0;
  const size_t runarr = size_t(d->bh) * nruns * (d->d == 64 ? O1Run<64>::RS : O1Run<32>::RS) * 4;
  const size_t runharr = size_t(d->bh) * nruns * d->d * d->d * 2;
  p.run = take(runarr); p.runh = take(runharr);
  p.keep_resid = p.save && d->dtype == FASTMAX_BF16 && !p.o1;
  p.ores = take(p.keep_resid ? size_t(d->bh) * p.npad_q * d->d * 2 : 0);
  p.fwd_bytes = off ? off : 256;
  off = 0;
  p.b_kt = take(tkt); p.b_vt = take(tkt); p.b_qt = take(tqt); p.b_qct = take(tqt);
  p.b_kr = take(tk); p.b_vr = take(tk); p.b_qr = take(tq);
  p.b_gh = take(tq); p.b_ght = take(tqt);
  p.b_cv = take(p.o1 ? 0 : size_t(d->bh) * p.npad_q * 4);
  p.b_bigq = take(bigarr); p.b_smallq = take(size_t(d->bh) * p.nslots * smallsz);
  p.b_bigk = take(bigarr); p.b_smallk = take(size_t(d->bh) * p.nslots * smallsz);
  p.b_bigv = take(p.o1 ? 0 : bigarr);
  p.b_gpart = take(p.half ? size_t(d->bh) * fm_grad_scale_blocks(d->nq) * 4 : 0);   // see k_grad_scale
  // parts of B = sum dy . y per workgroup of the dQ and dK kernels (128 own tokens at least), see k_norm_fix
  const bool jac = d->norm.grad != 0;
  p.b_bq = take(jac && d->norm.q_keys ? size_t(d->bh) * ((d->nq + 127) / 128) * 4 : 0);
  p.b_bk = take(jac && d->norm.k_keys ? size_t(d->bh) * ((d->nk + 127) / 128) * 4 : 0);
  p.b_runq = take(runarr); p.b_runqh = take(runharr); p.b_runk = take(runarr); p.b_runkh = take(runharr);
  p.bwd_bytes = off ? off : 256;
  return FASTMAX_OK;
}

template <typename T> TRef<const T> cref(const void* ptr, const FastmaxStrides& s) {
  return fm_ref<const T>(static_cast<const T*>(ptr), s);
}
template <typename T> TRef<T> mref(void* ptr, const FastmaxStrides& s) { return fm_ref<T>(static_cast<T*>(ptr), s); }

// k and v (same length) in one launch
template <typename TIO, typename E, int DH>
int launch_transpose2(const void* x0, const FastmaxStrides& s0, E* xt0, E* xr0, float scale0, const NormFold& f0,
                      const void* x1, const FastmaxStrides& s1, E* xt1, E* xr1, float scale1, const NormFold& f1, int bh,
                      int n, int npad, fm_stream_t stream) {
  const TransposeJob<TIO, E> j0{cref<TIO>(x0, s0), xt0, xr0, scale0, f0}, j1{cref<TIO>(x1, s1), xt1, xr1, scale1, f1};
  ProfScope prof(FM_K_TRANSPOSE, stream);
  FM_KERNEL_LAUNCH((k_transpose<TIO, E, DH>), fm_dim3(npad / 64, bh, 2), fm_dim3(FM_THREADS), 0, stream, j0, j1, n, npad);
  return fm_launch_status();
}

// per-segment sums -> prefix / suffix states (after a build whose workgroups took one step each)
template <typename E, int DH>
int launch_scan(const BuildArgs<E>& a, int bh, int nsteps, fm_stream_t stream) {
  constexpr int VE = 16 / sizeof(E);                            // 16-byte items, as k_state_scan counts them
  const int64_t nbig = (a.quad ? int64_t(DH + 1) * DH * DH : int64_t(DH) * DH) / VE;
  const int64_t total = nbig * (a.big2 ? 2 : 1) + (StateDims<DH>::SMALL - (a.quad ? 0 : DH * DH)) / 4;
  // one wavefront per workgroup: an order-1 scan is a thousand items per batch*head, and spread over
  // four times as many CUs each of them moves a quarter of the bytes
  FM_KERNEL_LAUNCH((k_state_scan<E, DH>), fm_dim3(int((total + FM_SCAN_THREADS - 1) / FM_SCAN_THREADS), bh),
                   fm_dim3(FM_SCAN_THREADS), 0, stream, a.big, a.big2, a.small, a.nslots, nsteps, a.mode, a.nseg, a.quad);
  return fm_launch_status();
}

template <typename E, int DH, int NA, int TT, int SPW, int KB>
int launch_build_cfg(const BuildArgs<E>& a, int groups, int bh, int nsteps, fm_stream_t stream) {
  constexpr int PT = TT + Mma<E>::PAD;
  constexpr int AW = 4 * NA;
  size_t lds = size_t(3 * DH + AW) * PT * sizeof(E);                        // staged token tiles
  const size_t red = size_t(SPW < 4 ? SPW : 4) * 4 * 64 * 16 * 4;                // reduction scratch of the lower-order tiles
  const size_t snap = size_t(AW) * DH * (DH + Mma<E>::PAD) * sizeof(E);      // snapshot staging
  if (lds < red) lds = red;
  if (lds < snap) lds = snap;
  // the _Float16 walk with a CU to itself keeps two buffers of token tiles and stages its stores behind them
  if (sizeof(E) == 2 && KB >= 4) lds = 2 * size_t(3 * DH + AW) * PT * sizeof(E) + (red > snap ? red : snap) + 16;   // + eight ones
  fm_allow_lds(reinterpret_cast<const void*>(&k_build<E, DH, NA, TT, SPW, KB>), lds);
  FM_KERNEL_LAUNCH((k_build<E, DH, NA, TT, SPW, KB>), fm_dim3(groups, bh, a.seg_parallel ? nsteps : 1),
                   fm_dim3(FM_THREADS), lds, stream, a);
  int st = fm_launch_status();
  if (st || !a.seg_parallel || nsteps < 2) return st;
  return launch_scan<E, DH>(a, bh, nsteps, stream);
}

template <typename E, int DH>
int launch_build(const BuildArgs<E>& args, int bh, fm_stream_t stream) {
  const int nsteps = args.mode == FM_WALK_TOTAL ? 1 : args.nseg - 1;
  if (nsteps <= 0) return FASTMAX_OK;
  ProfScope prof(FM_K_BUILD, stream);
  constexpr int NT = DH / 32, NSMALL = 2 * NT * NT + 2 * NT;
  BuildArgs<E> a = args;
  if (a.quad) {
    // One value of `a` per wavefront (4 per workgroup) and 64-token tiles: 64 accumulator
    // registers per wavefront leave room for two workgroups per CU, which measured faster on
    // MI355X than two values per wavefront at one workgroup per CU (0.092 vs 0.115 ms at
    // B*H = 32, N = 4096, D = 64).
    constexpr int G = DH / 4;
    a.seg_parallel = nsteps > 1 && bh * G < 256;
    if (a.seg_parallel) a.skip_big = 0;                // the scan that follows treats both copies alike
    // the one-workgroup-per-CU variant on _Float16: 128-token tiles, all eight k-steps of fragments requested at once
    constexpr int TTS = sizeof(E) == 2 ? 128 : 64;
    constexpr int KBS = sizeof(E) == 2 ? 8 : 4;
    // at most one workgroup per CU: all the registers are its own, every fragment of a tile is in flight at once
    if (bh * G * (a.seg_parallel ? nsteps : 1) <= 256)
      return launch_build_cfg<E, DH, 1, TTS, (NSMALL + G - 1) / G, KBS>(a, G, bh, nsteps, stream);
    return launch_build_cfg<E, DH, 1, 64, (NSMALL + G - 1) / G, 2>(a, G, bh, nsteps, stream);
  }
  // Order 1: the sums are a few 32x32 tiles per segment, far too little work per token tile for
  // a staged walk.  One workgroup per (segment, batch*head) sums its segment from fragments loaded
  // straight from the operands, and a scan over the segments follows.
  a.seg_parallel = 1;
  if (Mma<E>::HAS_TR && a.pr && a.mode != FM_WALK_TOTAL) {
    // row-major operands, transposing LDS reads: nobody had to write transposed copies (see k_build1_rows)
    const size_t ldsr = Build1RowsCfg<E, DH>::lds_bytes();
    fm_allow_lds(reinterpret_cast<const void*>(&k_build1_rows<E, DH>), ldsr);
    FM_KERNEL_LAUNCH((k_build1_rows<E, DH>), fm_dim3(1, bh, nsteps), fm_dim3(FM_THREADS), ldsr, stream, a);
    const int st = fm_launch_status();
    return (st || nsteps < 2) ? st : launch_scan<E, DH>(a, bh, nsteps, stream);
  }
  if (nsteps > 1) {
    // several segments: operand tiles staged through LDS, sum tiles dealt to the wavefronts (see k_build1_seg)
    const size_t lds1 = Build1Cfg<E, DH>::lds_bytes(a.zt != nullptr && a.za_sel == FM_SRC_Z);
    fm_allow_lds(reinterpret_cast<const void*>(&k_build1_seg<E, DH>), lds1);
    FM_KERNEL_LAUNCH((k_build1_seg<E, DH>), fm_dim3(1, bh, nsteps), fm_dim3(FM_THREADS), lds1, stream, a);
    const int st = fm_launch_status();
    return st ? st : launch_scan<E, DH>(a, bh, nsteps, stream);
  }
  const size_t lds = size_t(4) * 4 * 64 * 16 * 4;
  fm_allow_lds(reinterpret_cast<const void*>(&k_build1<E, DH>), lds);
  FM_KERNEL_LAUNCH((k_build1<E, DH>), fm_dim3(1, bh, nsteps), fm_dim3(FM_THREADS), lds, stream, a);
  return fm_launch_status();
}

// The order-2 walk held per value column (k_walk_sym), where the plan says so.
template <typename E, int DH> bool walk_sym_applies(const Plan& p, int, bool) { return sizeof(E) == 2 && DH == 64 && p.sym; }
inline int launch_walk_sym(const WalkSymArgs& a, int bh, fm_stream_t stream) {
  const int nsteps = a.mode == FM_WALK_TOTAL ? 1 : a.nseg - 1;
  if (nsteps <= 0) return FASTMAX_OK;
  ProfScope prof(FM_K_BUILD, stream);
  const size_t lds = WalkSymCfg<64>::lds_bytes();
  fm_allow_lds(reinterpret_cast<const void*>(&k_walk_sym<64>), lds);
  FM_KERNEL_LAUNCH((k_walk_sym<64>), fm_dim3(16, bh), fm_dim3(WalkSymCfg<64>::THREADS), lds, stream, a);
  return fm_launch_status();
}

// Dynamic LDS of a token kernel (kind 0: k_pv, 1: k_ds, 2: k_ds with dV, 3: k_ds with the fused
// preparation, 4: k_ds with dV and states): va, vb | own rows | region, where the dense stages and the output staging lie over
// the own rows and the region.
template <typename E, int DH, int QT> size_t tok_lds_bytes(int kind) {
  typedef TokCfg<E, DH, QT> C;
  size_t region = size_t(2) * (kind == 0 ? C::SLAB_SYM : C::SLAB) * sizeof(E);   // k_pv reads its states with fm_readout_sym
  const size_t zs = size_t(C::NZ) * DH * C::PS * sizeof(E);
  if (zs > region) region = zs;
  if (C::WIDE) region = 0;                             // no states at that width
  size_t body = size_t(C::QW) * C::PQ * sizeof(E) + region;
  const size_t outst = size_t(C::QW) * fm_store_pitch(DH) * 4;
  const size_t stage = kind == 0 ? size_t(2) * C::PV_STAGE * sizeof(E)
                                 : size_t(C::DS_NBUF) * (kind == 2 || kind == 4 ? C::DV_STAGE : C::DS_STAGE) * sizeof(E);
  if (kind == 4) body += size_t(C::QW) * (DH + 1) * 4;      // dK of the fused state readout, behind the slabs
  const size_t prep = size_t(2) * C::QW * C::PQ * sizeof(E) + size_t(C::QW) * 4;   // own q' rows, gh rows, c
  if (outst > body) body = outst;
  if (stage > body) body = stage;
  if (kind == 3 && prep > body) body = prep;
  return size_t(2 * DH) * 4 + body;
}

inline NormFold fold_of(const void* keys, int n, float lim) {
  return NormFold{static_cast<const unsigned long long*>(keys), fm_maxnorm_blocks(n), lim};
}
inline NormFold q_fold(const FastmaxDesc* d) { return fold_of(d->norm.q_keys, d->nq, d->norm.lim); }
inline NormFold k_fold(const FastmaxDesc* d) { return fold_of(d->norm.k_keys, d->nk, d->norm.lim); }
const NormFold no_fold{nullptr, 0, 1.0f};

template <typename TIO, typename E> void tok_common(TokArgs<TIO, E>& a, const FastmaxDesc* d, const Plan& p) {
  a.own_fold = no_fold; a.out_fold = no_fold; a.brows = nullptr; a.bpart = nullptr;
  a.own_io = TRef<const TIO>{nullptr, 0, 0, 0, 0, 0};
  a.own_r = nullptr; a.own2_r = nullptr; a.cv = nullptr; a.xr = nullptr; a.yr = nullptr; a.zt = nullptr; a.zt2 = nullptr; a.bigb = nullptr;
  a.out2 = TRef<TIO>{nullptr, 0, 0, 0, 0, 0}; a.out2_scale = 1.0f;
  a.g = TRef<float>{nullptr, 0, 0, 0, 0, 0};
  a.nslots = p.nslots; a.L = p.L; a.nseg = p.nseg; a.causal = d->mask != 0; a.use_state = p.use_state;
  a.quad = p.quad; a.a0 = p.a0; a.a1 = p.a1; a.a2 = p.a2; a.sc = p.sc; a.out_scale = 1.0f; a.zscale = 1.0f;
  a.own_o = TRef<const TIO>{nullptr, 0, 0, 0, 0, 0}; a.own_do = a.own_o;
  a.w_gh = nullptr; a.w_qr = nullptr; a.w_cv = nullptr; a.gpart = nullptr; a.gnblk = 0;
  a.out_resid = nullptr; a.own_ores = nullptr; a.state_xscale = 1.0f;
}

template <typename TIO, typename E, int DH, int QT, int OWN, int QF = 0>
int launch_pv(const TokArgs<TIO, E>& a, int bh, int kernel_id, fm_stream_t stream) {
  typedef TokCfg<E, DH, QT> C;
  const size_t lds = tok_lds_bytes<E, DH, QT>(0);
  fm_allow_lds(reinterpret_cast<const void*>(&k_pv<TIO, E, DH, QT, OWN, QF>), lds);
  ProfScope prof(kernel_id, stream);
  FM_KERNEL_LAUNCH((k_pv<TIO, E, DH, QT, OWN, QF>), fm_dim3((a.n_own + C::QW - 1) / C::QW, bh), fm_dim3(FM_THREADS), lds,
                   stream, a);
  return fm_launch_status();
}

template <typename TIO, typename E, int DH, int QT, int OWN, int DV = 0, int PREP = 0, int QF = 0, int STR = 0>
int launch_ds(const TokArgs<TIO, E>& a, int bh, int kernel_id, fm_stream_t stream) {
  typedef TokCfg<E, DH, QT> C;
  const size_t lds = tok_lds_bytes<E, DH, QT>(PREP ? 3 : (DV ? (a.use_state ? 4 : 2) : 1));
  fm_allow_lds(reinterpret_cast<const void*>(&k_ds<TIO, E, DH, QT, OWN, DV, PREP, QF, STR>), lds);
  ProfScope prof(kernel_id, stream);
  FM_KERNEL_LAUNCH((k_ds<TIO, E, DH, QT, OWN, DV, PREP, QF, STR>), fm_dim3((a.n_own + C::QW - 1) / C::QW, bh), fm_dim3(FM_THREADS), lds,
                   stream, a);
  return fm_launch_status();
}

// ---- order 1 in 128-token segments on the caller's tensors (fm_o1.h) -------------------------
// The sums inside every run of segments (QG = 0: keys and values, prefix walk; QG = 1: queries and gh, suffix
// walk), then the scan over the runs' totals.
template <typename TIO, int DH, int QG>
int launch_o1_sums(O1SumArgs<TIO>& a, fm_half* runhalf, int bh, fm_stream_t stream) {
  const int nruns = fm_o1_runs(a.b.nseg, a.run_len);
  ProfScope prof(FM_K_BUILD, stream);
  const size_t lds = fm_o1_sums_lds<DH>();
  fm_allow_lds(reinterpret_cast<const void*>(&k_o1_sums<TIO, DH, QG>), lds);
  FM_KERNEL_LAUNCH((k_o1_sums<TIO, DH, QG>), fm_dim3(1, bh, nruns), fm_dim3(FM_THREADS), lds, stream, a);
  const int st = fm_launch_status();
  if (st) return st;
  FM_KERNEL_LAUNCH((k_o1_runscan<DH>), fm_dim3((O1Run<DH>::RS + FM_THREADS - 1) / FM_THREADS, bh), fm_dim3(FM_THREADS), 0, stream,
                   a.runtot, runhalf, nruns, a.b.mode == FM_WALK_SUFFIX ? 1 : 0);
  return fm_launch_status();
}

// key / value sums of the forward (and of a backward that has no saved forward): big [v][k']
template <typename TIO, int DH>
int o1_key_sums(const FastmaxDesc* d, const Plan& p, const void* k, const void* v, fm_half* big, float* small,
                float* runtot, fm_half* runhalf, fm_stream_t stream) {
  O1SumArgs<TIO> a;
  a.x0 = cref<TIO>(k, d->sk); a.x1 = cref<TIO>(v, d->sv); a.o = a.x0; a.g = TRef<const float>{nullptr, 0, 0, 0, 0, 0};
  a.scale0 = p.sc; a.fold0 = k_fold(d); a.gpart = nullptr; a.gnblk = 0; a.n = d->nk; a.runtot = runtot; a.run_len = p.o1_run;
  BuildArgs<fm_half>& b = a.b;
  b.xt = nullptr; b.pt = nullptr; b.rt = nullptr; b.zt = nullptr; b.pr = nullptr; b.rr = nullptr; b.cw = nullptr;
  b.za_sel = FM_SRC_R; b.zb_sel = FM_SRC_R; b.vb_from_r = 0; b.seg_parallel = 1; b.skip_big = 0;
  b.npad = p.npad_k; b.nseg = p.nseg; b.L = p.L; b.mode = FM_WALK_PREFIX; b.quad = 0;
  b.big = big; b.big2 = nullptr; b.small = small; b.nslots = p.nslots;
  b.coef2 = 0.f; b.coef2b = 0.f; b.coefz = 0.f; b.coef1 = p.a1; b.coef1b = p.a1; b.coefva = p.a1; b.coefvb = p.a0;
  return launch_o1_sums<TIO, DH, 0>(a, runhalf, d->bh, stream);
}

template <typename TIO, int DH>
int run_forward_o1(const FastmaxDesc* d, const Plan& p, const void* q, const void* k, const void* v, void* o, float* g,
                   char* ws, fm_stream_t stream) {
  fm_half* big = reinterpret_cast<fm_half*>(ws + p.big);
  float* small = reinterpret_cast<float*>(ws + p.small);
  float* runtot = reinterpret_cast<float*>(ws + p.run);
  fm_half* runhalf = reinterpret_cast<fm_half*>(ws + p.runh);
  int st = o1_key_sums<TIO, DH>(d, p, k, v, big, small, runtot, runhalf, stream);   // the backward reads the same sums: nothing else to save
  if (st) return st;
  O1FwdArgs<TIO> a;
  a.q = cref<TIO>(q, d->sq); a.k = cref<TIO>(k, d->sk); a.v = cref<TIO>(v, d->sv);
  a.o = mref<TIO>(o, d->so); a.g = mref<float>(g, d->sg);
  a.n = d->nq; a.nseg = p.nseg; a.nslots = p.nslots; a.big = big; a.small = small;
  a.runbig = runhalf; a.runtot = runtot; a.run_len = p.o1_run; a.nruns = fm_o1_runs(p.nseg, p.o1_run);
  a.a0 = p.a0; a.a1 = p.a1; a.sc = p.sc; a.q_fold = q_fold(d); a.k_fold = k_fold(d);
  const size_t lds = fm_o1_fwd_lds<DH>();
  fm_allow_lds(reinterpret_cast<const void*>(&k_o1_fwd<TIO, DH>), lds);
  ProfScope prof(FM_K_FWD, stream);
  FM_KERNEL_LAUNCH((k_o1_fwd<TIO, DH>), fm_dim3(p.nseg, d->bh), fm_dim3(FM_THREADS), lds, stream, a);
  return fm_launch_status();
}

template <typename TIO, typename E, int DH, int QT>
int run_forward(const FastmaxDesc* d, const Plan& p, const void* q, const void* k, const void* v, void* o,
                float* g, char* ws, fm_stream_t stream) {
  if constexpr (sizeof(E) == 2 && DH <= 64) {
    if (p.o1) return run_forward_o1<TIO, DH>(d, p, q, k, v, o, g, ws, stream);
  }
  E* kt = reinterpret_cast<E*>(ws + p.kt);
  E* vt = reinterpret_cast<E*>(ws + p.vt);
  E* big = reinterpret_cast<E*>(ws + p.big);
  float* small = reinterpret_cast<float*>(ws + p.small);
  E* kr = reinterpret_cast<E*>(ws + p.kr);
  E* vr = (p.save || p.half) ? reinterpret_cast<E*>(ws + p.vr) : nullptr;
  // the transposed copies feed the state walk and the fp32 kernels; the _Float16 token kernels read
  // transposed fragments out of row tiles
  if (sizeof(E) == 2 && (!p.use_state || p.rows_build)) { kt = nullptr; vt = nullptr; }
  int st = launch_transpose2<TIO, E, DH>(v, d->sv, vt, vr, 1.0f, no_fold, k, d->sk, kt, kr, p.sc, k_fold(d), d->bh, d->nk,
                                         p.npad_k, stream);
  if (st) return st;
  if constexpr (DH <= 64) {
  if (p.use_state) {
    BuildArgs<E> b;
    b.seg_parallel = 0; b.skip_big = 0;
    b.xt = kt; b.pt = vt; b.rt = kt; b.zt = nullptr; b.za_sel = FM_SRC_R; b.zb_sel = FM_SRC_R;
    b.pr = p.rows_build ? vr : nullptr; b.rr = p.rows_build ? kr : nullptr; b.cw = nullptr;
    b.npad = p.npad_k; b.nseg = p.nseg; b.L = p.L; b.mode = d->mask ? FM_WALK_PREFIX : FM_WALK_TOTAL;
    b.quad = p.quad; b.big = big; b.small = small; b.nslots = p.nslots;
    // saved for the backward: the transposed tiles are the (k, k, v) state that dQ reads
    b.big2 = p.save ? reinterpret_cast<E*>(ws + p.big2) : nullptr;
    b.vb_from_r = 0; b.coef2b = 2.0f * p.a2; b.coef1b = p.a1;
    b.coef2 = p.a2; b.coef1 = p.a1; b.coefz = p.a2; b.coefva = p.a1; b.coefvb = p.a0;
    bool walked = false;
    if constexpr (sizeof(E) == 2) {
      if (walk_sym_applies<E, DH>(p, d->bh, d->mask != 0)) {
        // values = v, keys = k': one layout serves the forward, and the backward's dQ reads the same slabs transposed
        WalkSymArgs w;
        w.kt = kt; w.xt = vt; w.cw = nullptr; w.npad = p.npad_k; w.nseg = p.nseg; w.L = p.L; w.mode = b.mode; w.nslots = p.nslots;
        w.o2 = big; w.o1_vk = big; w.o1_kv = nullptr; w.small = small;
        w.coef2 = p.a2; w.coef1 = p.a1; w.coefz = p.a2; w.coefva = p.a1; w.coefvb = p.a0;
        st = launch_walk_sym(w, d->bh, stream);
        walked = true;
      }
    }
    if (!walked) st = launch_build<E, DH>(b, d->bh, stream);
    if (st) return st;
  }
  }
  TokArgs<TIO, E> a;
  tok_common(a, d, p);
  a.own_io = cref<TIO>(q, d->sq);
  a.own_fold = q_fold(d);
  a.xr = kr; a.yr = vr; a.zt = vt; a.npad_own = p.npad_q; a.npad_str = p.npad_k;
  a.big = big; a.small = small;
  a.out = mref<TIO>(o, d->so);
  a.g = mref<float>(g, d->sg);
  a.n_own = d->nq; a.n_str = d->nk;
  if (p.keep_resid) a.out_resid = reinterpret_cast<fm_half*>(ws + p.ores);
  // order-2 states: two tiles per wavefront halve the state bytes a token reads (forward 1.38 -> 0.94 ms
  // at B*H = 16, N = 65536 on MI355X); without states one tile per wavefront and more workgroups per CU win
  if constexpr (DH <= 64) {
    if (sizeof(E) == 2 && p.use_state && p.quad)
      return launch_pv<TIO, E, DH, (sizeof(E) == 2 ? 2 : QT), FM_OWN_Q>(a, d->bh, FM_K_FWD, stream);
  }
  if constexpr (sizeof(E) == 2 && DH <= 64) {
    if (p.qf) return launch_pv<TIO, E, DH, 1, FM_OWN_Q, 1>(a, d->bh, FM_K_FWD, stream);
  }
  return launch_pv<TIO, E, DH, QT, FM_OWN_Q>(a, d->bh, FM_K_FWD, stream);
}


// ---- causal with more keys than queries --------------------------------------------------
// Two ordinary problems on one workspace, one after the other on the same stream: the head
// (all queries, keys [0, nk - nq), unmasked) and the tail (keys [nk - nq, nk), causal, square).
struct SplitPlan {
  int off;                         // nk - nq
  FastmaxDesc head, head_b, tail;  // head_b: the head's backward (dq to a packed scratch tensor)
  size_t sub_fwd, sub_bwd;         // workspace of the larger of the two parts
  size_t off_a, off_ga, off_b;     // head's o and g (forward), head's dq (backward), after the parts' workspace
  size_t fwd_bytes, bwd_bytes;
};

inline bool is_split(const FastmaxDesc* d) { return d->mask && d->nk > d->nq; }

int make_split(const FastmaxDesc* d, SplitPlan& sp) {
  sp.off = d->nk - d->nq;
  const FastmaxStrides packed{int64_t(d->nq) * d->d, d->d, 0, 0, 0};
  sp.head = *d;
  sp.head.mask = 0; sp.head.nk = sp.off;
  sp.head.flags &= ~FASTMAX_FLAG_SAVE_FOR_BACKWARD;
  sp.head_b = sp.head;
  sp.head.so = packed;
  sp.head.sg = FastmaxStrides{d->nq, 1, 0, 0, 0};
  sp.head_b.sdq = packed;
  sp.tail = *d;
  sp.tail.nk = d->nq;
  sp.tail.flags &= ~FASTMAX_FLAG_SAVE_FOR_BACKWARD;
  Plan ph, pt;
  int st = make_plan(&sp.head, ph);
  if (st) return st;
  st = make_plan(&sp.tail, pt);
  if (st) return st;
  const size_t esz = d->dtype == FASTMAX_BF16 ? 2 : 4;
  const size_t rows = align256(size_t(d->bh) * d->nq * d->d * esz);
  sp.sub_fwd = align256(ph.fwd_bytes > pt.fwd_bytes ? ph.fwd_bytes : pt.fwd_bytes);
  sp.sub_bwd = align256(ph.bwd_bytes > pt.bwd_bytes ? ph.bwd_bytes : pt.bwd_bytes);
  sp.off_a = sp.sub_fwd;
  sp.off_ga = sp.off_a + rows;
  sp.fwd_bytes = sp.off_ga + align256(size_t(d->bh) * d->nq * 4);
  sp.off_b = sp.sub_bwd;
  sp.bwd_bytes = sp.off_b + rows;
  return FASTMAX_OK;
}

template <typename TIO, int DH>
int merge_parts(const FastmaxDesc* d, const SplitPlan& sp, const void* oa, const float* ga, void* o, float* g,
                fm_stream_t stream) {
  const TRef<const TIO> oar = cref<TIO>(oa, sp.head.so);
  const TRef<const float> gar = cref<float>(ga, sp.head.sg);
  const TRef<float> gr = mref<float>(g, d->sg);
  const int64_t items = int64_t(d->nq) * (DH / 8);
  FM_KERNEL_LAUNCH((k_merge_parts<TIO, DH>), fm_dim3(int((items + 255) / 256), d->bh), fm_dim3(256), 0, stream, oar, gar,
                   mref<TIO>(o, d->so), gr, d->nq);
  FM_KERNEL_LAUNCH(k_merge_denominators, fm_dim3((d->nq + 255) / 256, d->bh), fm_dim3(256), 0, stream, gar, gr, d->nq);
  return fm_launch_status();
}

template <typename TIO, int DH>
int add_rows(const FastmaxDesc* d, const SplitPlan& sp, const void* dqa, void* dq, fm_stream_t stream) {
  const int64_t items = int64_t(d->nq) * (DH / 8);
  FM_KERNEL_LAUNCH((k_add_rows<TIO, DH>), fm_dim3(int((items + 255) / 256), d->bh), fm_dim3(256), 0, stream,
                   cref<TIO>(dqa, sp.head_b.sdq), mref<TIO>(dq, d->sdq), d->nq);
  return fm_launch_status();
}

}  // namespace

#include "fastmax_api_bwd.inc"

extern "C" {

int fastmax_version(void) { return 300; }   // 0.3.0: heads of 128 (bf16), the decoding state in its symmetric column-block layout (a state of 0.2.x is not readable), bench aids out of the product library

const char* fastmax_status_string(int status) {
  switch (status) {
    case FASTMAX_OK: return "ok";
    case FASTMAX_ERR_NULL: return "null pointer";
    case FASTMAX_ERR_SHAPE: return "invalid shape or strides";
    case FASTMAX_ERR_UNSUPPORTED: return "unsupported configuration (d must be 32 or 64, p 1 or 2, masked needs nq <= nk)";
    case FASTMAX_ERR_WORKSPACE: return "workspace missing, too small or not 256-byte aligned";
    case FASTMAX_ERR_LAUNCH: return "HIP launch failed";
    case FASTMAX_ERR_DTYPE: return "unknown dtype";
    case FASTMAX_ERR_TOO_LARGE: return "problem needs more scratch than the library's static buffer holds";
    default: return "unknown status";
  }
}

int fastmax_workspace_bytes(const FastmaxDesc* desc, size_t* forward_bytes, size_t* backward_bytes) {
  int st = validate(desc);
  if (st) return st;
  size_t f = 0, b = 0;
  if (is_split(desc)) {
    SplitPlan sp;
    st = make_split(desc, sp);
    f = sp.fwd_bytes; b = sp.bwd_bytes;
  } else {
    Plan p;
    st = make_plan(desc, p);
    f = p.fwd_bytes; b = p.bwd_bytes;
  }
  if (st) return st;
  if (forward_bytes) *forward_bytes = f;
  if (backward_bytes) *backward_bytes = b;
  return FASTMAX_OK;
}

static int forward_one(const FastmaxDesc* desc, const void* q, const void* k, const void* v, void* o, float* g,
                       void* workspace, size_t workspace_bytes, void* hip_stream) {
  Plan p;
  int st = make_plan(desc, p);
  if (st) return st;
  if (!q || !k || !v || !o || !g) return FASTMAX_ERR_NULL;
  if (!strides_ok(desc->sq, desc->bh, desc->nq, desc->d) || !strides_ok(desc->sk, desc->bh, desc->nk, desc->d) ||
      !strides_ok(desc->sv, desc->bh, desc->nk, desc->d) || !strides_ok(desc->so, desc->bh, desc->nq, desc->d) ||
      !strides_ok(desc->sg, desc->bh, desc->nq, 1))
    return FASTMAX_ERR_SHAPE;
  if (!workspace || workspace_bytes < p.fwd_bytes || reinterpret_cast<uintptr_t>(workspace) % 256)
    return FASTMAX_ERR_WORKSPACE;
  char* ws = static_cast<char*>(workspace);
  fm_stream_t stream = static_cast<fm_stream_t>(hip_stream);
  if (p.half) {
    if (desc->d == FM_WIDE_HEAD) return run_forward<fm_bf16, fm_half, FM_WIDE_HEAD, 1>(desc, p, q, k, v, o, g, ws, stream);
    if (desc->d == 64) return run_forward<fm_bf16, fm_half, 64, 1>(desc, p, q, k, v, o, g, ws, stream);
    return run_forward<fm_bf16, fm_half, 32, 1>(desc, p, q, k, v, o, g, ws, stream);
  }
  if (desc->dtype == FASTMAX_BF16) {               // bf16 tensors, fp32 arithmetic (FASTMAX_FLAG_F32_COMPUTE)
    if (desc->d == 64) return run_forward<fm_bf16, float, 64, 1>(desc, p, q, k, v, o, g, ws, stream);
    return run_forward<fm_bf16, float, 32, 1>(desc, p, q, k, v, o, g, ws, stream);
  }
  if (desc->d == 64) return run_forward<float, float, 64, 1>(desc, p, q, k, v, o, g, ws, stream);
  return run_forward<float, float, 32, 1>(desc, p, q, k, v, o, g, ws, stream);
}

int fastmax_forward(const FastmaxDesc* desc, const void* q, const void* k, const void* v, void* o, float* g,
                    void* workspace, size_t workspace_bytes, void* hip_stream) {
  const int st = validate(desc);
  if (st) return st;
  if (!is_split(desc)) return forward_one(desc, q, k, v, o, g, workspace, workspace_bytes, hip_stream);
  // causal with nk > nq: the keys every query sees, then the square causal part, then the merge
  SplitPlan sp;
  int s2 = make_split(desc, sp);
  if (s2) return s2;
  if (!q || !k || !v || !o || !g) return FASTMAX_ERR_NULL;
  if (!strides_ok(desc->sk, desc->bh, desc->nk, desc->d) || !strides_ok(desc->sv, desc->bh, desc->nk, desc->d))
    return FASTMAX_ERR_SHAPE;
  if (!workspace || workspace_bytes < sp.fwd_bytes || reinterpret_cast<uintptr_t>(workspace) % 256)
    return FASTMAX_ERR_WORKSPACE;
  char* ws = static_cast<char*>(workspace);
  void* oa = ws + sp.off_a;
  float* ga = reinterpret_cast<float*>(ws + sp.off_ga);
  s2 = forward_one(&sp.head, q, k, v, oa, ga, ws, sp.sub_fwd, hip_stream);
  if (s2) return s2;
  const size_t esz = desc->dtype == FASTMAX_BF16 ? 2 : 4;
  const char* kt = static_cast<const char*>(k) + size_t(sp.off) * desc->sk.n * esz;
  const char* vt = static_cast<const char*>(v) + size_t(sp.off) * desc->sv.n * esz;
  s2 = forward_one(&sp.tail, q, kt, vt, o, g, ws, sp.sub_fwd, hip_stream);
  if (s2) return s2;
  fm_stream_t stream = static_cast<fm_stream_t>(hip_stream);
  if (desc->dtype == FASTMAX_BF16)
    return desc->d == 64 ? merge_parts<fm_bf16, 64>(desc, sp, oa, ga, o, g, stream) : merge_parts<fm_bf16, 32>(desc, sp, oa, ga, o, g, stream);
  return desc->d == 64 ? merge_parts<float, 64>(desc, sp, oa, ga, o, g, stream) : merge_parts<float, 32>(desc, sp, oa, ga, o, g, stream);
}

int fastmax_forward_static(const FastmaxDesc* desc, const void* q, const void* k, const void* v, void* o, float* g,
                           void* hip_stream) {
  size_t need = 0;
  const int st = fastmax_workspace_bytes(desc, &need, nullptr);
  if (st) return st;
  if (need > size_t(FASTMAX_STATIC_SCRATCH_BYTES)) return FASTMAX_ERR_TOO_LARGE;
  void* ws = nullptr;
  const int sa = fm_static_scratch(&ws);
  if (sa) return sa;
  // nothing in the scratch has to start at zero: every kernel of the forward writes what a later one reads
  return fastmax_forward(desc, q, k, v, o, g, ws, size_t(FASTMAX_STATIC_SCRATCH_BYTES), hip_stream);
}

static int backward_one(const FastmaxDesc* desc, const void* q, const void* k, const void* v, const void* o,
                        const float* g, const void* d_o, void* dq, void* dk, void* dv, const void* fwd_ws,
                        size_t fwd_ws_bytes, void* workspace, size_t workspace_bytes, void* hip_stream) {
  Plan p;
  int st = make_plan(desc, p);
  if (st) return st;
  if (!q || !k || !v || !o || !g || !d_o || !dq || !dk || !dv) return FASTMAX_ERR_NULL;
  if (!strides_ok(desc->sq, desc->bh, desc->nq, desc->d) || !strides_ok(desc->sk, desc->bh, desc->nk, desc->d) ||
      !strides_ok(desc->sv, desc->bh, desc->nk, desc->d) || !strides_ok(desc->so, desc->bh, desc->nq, desc->d) ||
      !strides_ok(desc->sg, desc->bh, desc->nq, 1) || !strides_ok(desc->sdo, desc->bh, desc->nq, desc->d) ||
      !strides_ok(desc->sdq, desc->bh, desc->nq, desc->d) || !strides_ok(desc->sdk, desc->bh, desc->nk, desc->d) ||
      !strides_ok(desc->sdv, desc->bh, desc->nk, desc->d))
    return FASTMAX_ERR_SHAPE;
  if (!workspace || workspace_bytes < p.bwd_bytes || reinterpret_cast<uintptr_t>(workspace) % 256)
    return FASTMAX_ERR_WORKSPACE;
  if (fwd_ws) {
    if (!p.save) return FASTMAX_ERR_SHAPE;          // desc must carry the flag the forward was run with
    if (fwd_ws_bytes < p.fwd_bytes || reinterpret_cast<uintptr_t>(fwd_ws) % 256) return FASTMAX_ERR_WORKSPACE;
  }
  char* ws = static_cast<char*>(workspace);
  const char* fws = static_cast<const char*>(fwd_ws);
  fm_stream_t stream = static_cast<fm_stream_t>(hip_stream);
  if (p.half) {
    if (desc->d == FM_WIDE_HEAD) return run_backward_wide<fm_bf16, fm_half, FM_WIDE_HEAD>(desc, p, q, k, v, o, g, d_o, dq, dk, dv, fws, ws, stream);
    if (desc->d == 64) return run_backward<fm_bf16, fm_half, 64, 1>(desc, p, q, k, v, o, g, d_o, dq, dk, dv, fws, ws, stream);
    return run_backward<fm_bf16, fm_half, 32, 1>(desc, p, q, k, v, o, g, d_o, dq, dk, dv, fws, ws, stream);
  }
  if (desc->dtype == FASTMAX_BF16) {
    if (desc->d == 64) return run_backward<fm_bf16, float, 64, 1>(desc, p, q, k, v, o, g, d_o, dq, dk, dv, fws, ws, stream);
    return run_backward<fm_bf16, float, 32, 1>(desc, p, q, k, v, o, g, d_o, dq, dk, dv, fws, ws, stream);
  }
  if (desc->d == 64) return run_backward<float, float, 64, 1>(desc, p, q, k, v, o, g, d_o, dq, dk, dv, fws, ws, stream);
  return run_backward<float, float, 32, 1>(desc, p, q, k, v, o, g, d_o, dq, dk, dv, fws, ws, stream);
}

static int backward_impl(const FastmaxDesc* desc, const void* q, const void* k, const void* v, const void* o,
                         const float* g, const void* d_o, void* dq, void* dk, void* dv, const void* fwd_ws,
                         size_t fwd_ws_bytes, void* workspace, size_t workspace_bytes, void* hip_stream) {
  const int st = validate(desc);
  if (st) return st;
  if (!is_split(desc))
    return backward_one(desc, q, k, v, o, g, d_o, dq, dk, dv, fwd_ws, fwd_ws_bytes, workspace, workspace_bytes, hip_stream);
  // causal with nk > nq: both parts take the final o and g; dk and dv of the two parts are
  // disjoint key ranges, dq is their sum.  The forward keeps nothing for this case.
  if (fwd_ws) return FASTMAX_ERR_UNSUPPORTED;
  SplitPlan sp;
  int s2 = make_split(desc, sp);
  if (s2) return s2;
  if (!q || !k || !v || !o || !g || !d_o || !dq || !dk || !dv) return FASTMAX_ERR_NULL;
  if (!strides_ok(desc->sk, desc->bh, desc->nk, desc->d) || !strides_ok(desc->sv, desc->bh, desc->nk, desc->d) ||
      !strides_ok(desc->sdk, desc->bh, desc->nk, desc->d) || !strides_ok(desc->sdv, desc->bh, desc->nk, desc->d))
    return FASTMAX_ERR_SHAPE;
  if (!workspace || workspace_bytes < sp.bwd_bytes || reinterpret_cast<uintptr_t>(workspace) % 256)
    return FASTMAX_ERR_WORKSPACE;
  char* ws = static_cast<char*>(workspace);
  void* dqa = ws + sp.off_b;
  const size_t esz = desc->dtype == FASTMAX_BF16 ? 2 : 4;
  s2 = backward_one(&sp.head_b, q, k, v, o, g, d_o, dqa, dk, dv, nullptr, 0, ws, sp.sub_bwd, hip_stream);
  if (s2) return s2;
  const size_t ko = size_t(sp.off) * desc->sk.n * esz, vo = size_t(sp.off) * desc->sv.n * esz;
  const size_t dko = size_t(sp.off) * desc->sdk.n * esz, dvo = size_t(sp.off) * desc->sdv.n * esz;
  s2 = backward_one(&sp.tail, q, static_cast<const char*>(k) + ko, static_cast<const char*>(v) + vo, o, g, d_o, dq,
                    static_cast<char*>(dk) + dko, static_cast<char*>(dv) + dvo, nullptr, 0, ws, sp.sub_bwd, hip_stream);
  if (s2) return s2;
  fm_stream_t stream = static_cast<fm_stream_t>(hip_stream);
  if (desc->dtype == FASTMAX_BF16)
    return desc->d == 64 ? add_rows<fm_bf16, 64>(desc, sp, dqa, dq, stream) : add_rows<fm_bf16, 32>(desc, sp, dqa, dq, stream);
  return desc->d == 64 ? add_rows<float, 64>(desc, sp, dqa, dq, stream) : add_rows<float, 32>(desc, sp, dqa, dq, stream);
}

int fastmax_backward(const FastmaxDesc* desc, const void* q, const void* k, const void* v, const void* o,
                     const float* g, const void* d_o, void* dq, void* dk, void* dv, void* workspace,
                     size_t workspace_bytes, void* hip_stream) {
  return backward_impl(desc, q, k, v, o, g, d_o, dq, dk, dv, nullptr, 0, workspace, workspace_bytes, hip_stream);
}

int fastmax_backward_saved(const FastmaxDesc* desc, const void* q, const void* k, const void* v, const void* o,
                           const float* g, const void* d_o, void* dq, void* dk, void* dv,
                           const void* forward_workspace, size_t forward_workspace_bytes, void* workspace,
                           size_t workspace_bytes, void* hip_stream) {
  if (!forward_workspace) return FASTMAX_ERR_NULL;
  return backward_impl(desc, q, k, v, o, g, d_o, dq, dk, dv, forward_workspace, forward_workspace_bytes, workspace,
                       workspace_bytes, hip_stream);
}

size_t fastmax_normalize_stats_bytes(const FastmaxNormDesc* desc) {
  if (!desc || desc->bh <= 0 || desc->n <= 0 || desc->d <= 0) return 0;
  return size_t(desc->bh) * size_t(fm_norm_stride(desc->d, desc->n, desc->centre)) * sizeof(float);
}

int fastmax_normalize(const FastmaxNormDesc* desc, const void* x, void* y, float* stats, void* hip_stream) {
  ProfScope prof(FM_K_NORM, static_cast<fm_stream_t>(hip_stream));   // the whole pass (its kernels together)
  return fm_normalize_dispatch(desc, x, y, stats, static_cast<fm_stream_t>(hip_stream));
}

int fastmax_key_rpe(const FastmaxNormDesc* desc, const void* k, const float* rpe, void* k_out, float temperature,
                    void* hip_stream) {
  if (!(temperature > 0.0f) || !(temperature < 3.0e38f)) return FASTMAX_ERR_SHAPE;
  PointwiseArgs a;
  a.n = desc ? desc->n : 0; a.mode = 0; a.factor = temperature; a.table = rpe;
  return fm_pointwise_dispatch(desc, k, nullptr, k_out, a, static_cast<fm_stream_t>(hip_stream));
}

int fastmax_output_noise(const FastmaxNormDesc* desc, const void* o, const void* noise, void* o_out, float scale,
                         void* hip_stream) {
  if (!(scale == scale) || scale > 3.0e38f || scale < -3.0e38f) return FASTMAX_ERR_SHAPE;
  PointwiseArgs a;
  a.n = desc ? desc->n : 0; a.mode = 1; a.factor = scale; a.table = nullptr;
  return fm_pointwise_dispatch(desc, o, noise, o_out, a, static_cast<fm_stream_t>(hip_stream));
}

static int decode_validate(const FastmaxDesc* d) {
  if (!d) return FASTMAX_ERR_NULL;
  if (d->dtype != FASTMAX_F32 && d->dtype != FASTMAX_BF16) return FASTMAX_ERR_DTYPE;
  if (d->bh <= 0 || d->bh > 65535) return FASTMAX_ERR_SHAPE;
  if (d->p != 1 && d->p != 2) return FASTMAX_ERR_UNSUPPORTED;
  if (d->d != 32 && d->d != 64) return FASTMAX_ERR_UNSUPPORTED;
  if (!(d->inv_tau > 0.0f) || !(d->inv_tau < 3.0e38f)) return FASTMAX_ERR_SHAPE;
  return FASTMAX_OK;
}

size_t fastmax_decode_state_bytes(const FastmaxDesc* desc) {
  if (decode_validate(desc)) return 0;
  return size_t(desc->bh) * size_t(fm_decode_state_floats(desc->d, desc->p == 2 && desc->a2 != 0.0f)) * 4;
}

size_t fastmax_decode_scratch_bytes(const FastmaxDesc* desc) {
  if (decode_validate(desc)) return 0;
  return 256;      // a step is one launch that leaves nothing in memory between kernels: the scratch is not used any more
}

int fastmax_decode_absorb(const FastmaxDesc* desc, const void* k, const void* v, float* state, void* hip_stream) {
  const int st = decode_validate(desc);
  if (st) return st;
  if (!k || !v || !state) return FASTMAX_ERR_NULL;
  if (desc->nk <= 0 || desc->nk > (1 << 30)) return FASTMAX_ERR_SHAPE;
  if (!strides_ok(desc->sk, desc->bh, desc->nk, desc->d) || !strides_ok(desc->sv, desc->bh, desc->nk, desc->d))
    return FASTMAX_ERR_SHAPE;
  return fm_decode_dispatch(desc, nullptr, k, v, desc->nk, state, nullptr, nullptr, nullptr, static_cast<fm_stream_t>(hip_stream));
}

int fastmax_decode_step(const FastmaxDesc* desc, const void* q, const void* k, const void* v, float* state, void* o, float* g,
                        float* scratch, void* hip_stream) {
  const int st = decode_validate(desc);
  if (st) return st;
  if (!q || !k || !v || !state || !o || !g) return FASTMAX_ERR_NULL;
  if (!strides_ok(desc->sq, desc->bh, 1, desc->d) || !strides_ok(desc->sk, desc->bh, 1, desc->d) ||
      !strides_ok(desc->sv, desc->bh, 1, desc->d) || !strides_ok(desc->so, desc->bh, 1, desc->d) ||
      !strides_ok(desc->sg, desc->bh, 1, 1))
    return FASTMAX_ERR_SHAPE;
  return fm_decode_dispatch(desc, q, k, v, 1, state, o, g, scratch, static_cast<fm_stream_t>(hip_stream));
}

size_t fastmax_maxnorm_stats_bytes(int32_t bh, int32_t n) {
  if (bh <= 0 || n <= 0) return 0;
  return size_t(bh) * size_t(fm_maxnorm_blocks(n)) * 8;
}

int fastmax_maxnorm_stats(const FastmaxNormDesc* desc0, const void* x0, void* keys0, const FastmaxNormDesc* desc1,
                          const void* x1, void* keys1, void* hip_stream) {
  if (!desc0 || !x0 || !keys0) return FASTMAX_ERR_NULL;
  const bool two = desc1 != nullptr;
  if (two && (!x1 || !keys1)) return FASTMAX_ERR_NULL;
  for (const FastmaxNormDesc* d : {desc0, desc1}) {
    if (!d) continue;
    if (d->dtype != FASTMAX_F32 && d->dtype != FASTMAX_BF16) return FASTMAX_ERR_DTYPE;
    if (d->bh <= 0 || d->n <= 0 || d->bh > 65535 || d->n > (1 << 30)) return FASTMAX_ERR_SHAPE;
    if (d->d != 32 && d->d != 64) return FASTMAX_ERR_UNSUPPORTED;
    if (d->sx.n < d->d && d->n > 1) return FASTMAX_ERR_SHAPE;
  }
  if (two && (desc1->bh != desc0->bh || desc1->d != desc0->d || desc1->dtype != desc0->dtype)) return FASTMAX_ERR_SHAPE;
  if ((reinterpret_cast<uintptr_t>(keys0) | reinterpret_cast<uintptr_t>(keys1)) % 8) return FASTMAX_ERR_WORKSPACE;
  fm_stream_t stream = static_cast<fm_stream_t>(hip_stream);
  ProfScope prof(FM_K_NORM, stream);
  return fm_maxnorm_dispatch(desc0, x0, keys0, desc1, x1, keys1, stream);
}

size_t fastmax_normalize_backward_stats_bytes(const FastmaxNormDesc* desc) {
  if (!desc || desc->bh <= 0 || desc->n <= 0 || desc->d <= 0) return 0;
  return size_t(desc->bh) * size_t(fm_normb_stride(desc->d, desc->n, desc->centre)) * sizeof(float);
}

int fastmax_normalize_backward(const FastmaxNormDesc* desc, const void* x, const void* dy, void* dx, float* stats,
                               void* hip_stream) {
  ProfScope prof(FM_K_NORM, static_cast<fm_stream_t>(hip_stream));
  return fm_normalize_bwd_dispatch(desc, x, dy, dx, stats, static_cast<fm_stream_t>(hip_stream));
}

int fastmax_probe_mfma(float* out_f16, float* out_f32, void* hip_stream) {
  if (!out_f16 || !out_f32) return FASTMAX_ERR_NULL;
  FM_KERNEL_LAUNCH(k_probe_mfma, fm_dim3(1), fm_dim3(64), 0, static_cast<fm_stream_t>(hip_stream), out_f16, out_f32);
  return fm_launch_status();
}

int fastmax_probe_lds_transpose(float* out, void* hip_stream) {
  if (!out) return FASTMAX_ERR_NULL;
  FM_KERNEL_LAUNCH(k_probe_lds_tr, fm_dim3(1), fm_dim3(64), 0, static_cast<fm_stream_t>(hip_stream), out);
  return fm_launch_status();
}

#if defined(FM_BENCH_AIDS) && !defined(FM_HOSTSIM)
int fastmax_profile_begin(void) {
  for (auto& r : g_prof) { hipEventDestroy(r.a); hipEventDestroy(r.b); }
  g_prof.clear();
  g_prof_on = true;
  return FASTMAX_OK;
}

int fastmax_profile_end(int* kernel_ids, float* milliseconds, int capacity) {
  int n = 0;
  g_prof_on = false;
  for (auto& r : g_prof) {
    hipEventSynchronize(r.b);
    float ms = 0.f;
    hipEventElapsedTime(&ms, r.a, r.b);
    if (n < capacity) { if (kernel_ids) kernel_ids[n] = r.id; if (milliseconds) milliseconds[n] = ms; }
    ++n;
    hipEventDestroy(r.a); hipEventDestroy(r.b);
  }
  g_prof.clear();
  return n;
}

int fastmax_probe_mfma_rate(int workgroups, int iters, float* out, void* hip_stream) {
  if (!out) return FASTMAX_ERR_NULL;
  if (workgroups <= 0 || workgroups > 65536 || iters <= 0 || iters > (1 << 20)) return FASTMAX_ERR_SHAPE;
  FM_KERNEL_LAUNCH(k_probe_mfma_rate, fm_dim3(workgroups), fm_dim3(FM_THREADS), 0, static_cast<fm_stream_t>(hip_stream),
                   out, iters);
  return fm_launch_status();
}

int fastmax_probe_mix_rate(int workgroups, int iters, int own_tiles, float* out, void* hip_stream) {
  if (!out) return FASTMAX_ERR_NULL;
  if (workgroups <= 0 || workgroups > 65536 || iters <= 0 || iters > (1 << 20)) return FASTMAX_ERR_SHAPE;
  if (own_tiles != 1 && own_tiles != 2) return FASTMAX_ERR_UNSUPPORTED;
  fm_stream_t st = static_cast<fm_stream_t>(hip_stream);
  if (own_tiles == 1) FM_KERNEL_LAUNCH(k_probe_mix<1>, fm_dim3(workgroups), fm_dim3(FM_THREADS), 0, st, out, iters);
  else FM_KERNEL_LAUNCH(k_probe_mix<2>, fm_dim3(workgroups), fm_dim3(FM_THREADS), 0, st, out, iters);
  return fm_launch_status();
}

#endif  // FM_BENCH_AIDS

}  // extern "C"
