/* C ABI of libfastmax_hip.so: the Fastmax attention hot path on MI355X (gfx950).
 *
 * Plain pointers and sizes only; no torch types.  Every entry point enqueues
 * work on the given HIP stream and returns without synchronising.  Inputs are
 * never written.  All functions are re-entrant; the library keeps no mutable
 * global state besides per-kernel launch attributes.
 *
 * Tensors are addressed as (bh, n, d) through two element strides per tensor
 * (the feature axis is contiguous), so the reference extension's (n, bh, d)
 * layout and the model's (b, h, n, d) layout are both accepted without copies.
 */
#ifndef FASTMAX_HIP_H_
#define FASTMAX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  FASTMAX_OK = 0,
  FASTMAX_ERR_NULL = 1,          /* a required pointer is null */
  FASTMAX_ERR_SHAPE = 2,         /* sizes or strides are not valid */
  FASTMAX_ERR_UNSUPPORTED = 3,   /* valid, but not implemented (head size, order, masked nq > nk) */
  FASTMAX_ERR_WORKSPACE = 4,     /* workspace missing, too small or misaligned */
  FASTMAX_ERR_LAUNCH = 5,        /* the HIP runtime refused a launch */
  FASTMAX_ERR_DTYPE = 6,         /* unknown element type */
  FASTMAX_ERR_TOO_LARGE = 7      /* fastmax_forward_static: the problem needs more scratch than the static buffer */
};

enum { FASTMAX_F32 = 0, FASTMAX_BF16 = 1 };

/* flags */
enum {
  FASTMAX_FLAG_FORCE_MOMENTS = 1,   /* unmasked: always use the moment (linear-time) path */
  FASTMAX_FLAG_FORCE_DENSE = 2,     /* never build moment states (quadratic-time path) */
  FASTMAX_FLAG_SAVE_FOR_BACKWARD = 4, /* forward: also leave in its workspace what the backward of the same
                                        problem can reuse (converted k, v and the key-side moment states);
                                        forward_bytes grows accordingly */
  FASTMAX_FLAG_F32_COMPUTE = 8       /* bf16 tensors: do all arithmetic in fp32 (matrix products included)
                                        instead of _Float16; for inputs outside the range stated below.
                                        Many times slower; workspace sizes grow.  Ignored for fp32 tensors. */
};

/* Numeric range of the bf16 interface.  bf16 tensors are computed in _Float16 with fp32 accumulation
 * (the order-2 operands k_a * k_b have to be formed on the fly, and gfx950 has packed half
 * multiplies but no packed bf16 arithmetic).  _Float16 has 11 significand bits (bf16: 8) but a
 * narrow exponent: values beyond 65504 become infinities and values below 6e-5 lose precision.
 * Supported: |s_ij| = |q_i . k_j| * inv_tau <= 250 for every pair (so that a2 * s^2 <= 65504 / 2 for
 * a2 = 1/2; in general |a1 s| + |a2| s^2 < 6e4), |q|, |k| * sqrt(inv_tau) <= 6e4, and values v whose
 * entries lie between about 1e-4 and 1e2 in magnitude (the backward forms (dO / g) . v with dO / g brought to
 * [32, 64), and the moment states sum k k v over a segment, both rounded to _Float16; at 1e3 the gradients of q
 * and k, at 1e4 also the outputs of segmented sequences turn non-finite).  The reference model's normalised q and k (|q_i|, |k_j| <=
 * lim, transformer/model.py:97-102) satisfy this by construction.  Nothing saturates: an input
 * beyond the range turns into infinities that reach the outputs as inf / NaN rather than as finite
 * wrong numbers.  FASTMAX_FLAG_F32_COMPUTE lifts the limits at fp32 speed.  The size of dO is free (the
 * backward rescales dO / g per batch*head to the _Float16 range and back).  The 2e-2 accuracy of this
 * path also rests on weights f(s) that add up without cancelling, as the Taylor weights do (f > 0):
 * with a0 <= 0 the library computes bf16 tensors in fp32 on its own, as if the flag were set. */

/* Where slice i of the batch*head axis, token t, feature f of a tensor lives:
 *   heads <= 1:  i * bh + t * n + f
 *   heads  > 1:  (i / heads) * b + (i % heads) * bh + t * n + f      (i = batch * heads + head)
 * The second form takes the (b, n, h*d) output of a projection, viewed as (b, h, n, d), as it is:
 * b = n*h*d, bh = d, n = h*d (reference transformer/model.py:283-285 makes that view and the
 * reference wrapper then copies it, model.py:29-32). */
typedef struct FastmaxStrides {
  int64_t bh;     /* elements between consecutive batch*head slices (heads <= 1) or heads (heads > 1) */
  int64_t n;      /* elements between consecutive tokens */
  int64_t b;      /* elements between consecutive batches; read only when heads > 1 */
  int32_t heads;  /* heads per batch for the two-level form; 0 or 1: one stride for the whole axis */
  int32_t reserved;
} FastmaxStrides;

/* Optional: the max-norm normalisation of q and k (x_hat = lim * x / max_n ||x_n||_2 per batch*head,
 * reference transformer/model.py:97-102, the `normalize` flag of forwardpass) folded into the kernels'
 * loads instead of a pass that rewrites the tensors (reference apply_norm, fastmax_cuda_forward.cu:326-338).
 * q_keys / k_keys: device buffers written by fastmax_maxnorm_stats for the same q / k (null: that tensor is
 * used as it is).  grad (backward only): zero -> dq and dk are the gradients with respect to the normalised
 * tensors, which is what the reference's extension returns (its backward has no counterpart of apply_norm);
 * non-zero -> with respect to the raw q and k, the normalisation's own Jacobian included (what the
 * reference's Python variants get from autograd, score_function.py:40-55).  Not available for masked
 * problems with nk > nq. */
typedef struct FastmaxNormFold {
  const void* q_keys;
  const void* k_keys;
  float lim;
  int32_t grad;
} FastmaxNormFold;

/* Problem description shared by forward and backward.
 * Score s_ij = (q_i . k_j) * inv_tau;  weight f(s) = a0 + a1 s + a2 s^2 (a2 ignored when p == 1);
 * mask != 0: causal with nq <= nk, query i sees keys 0 .. nk - nq + i (the queries are aligned to
 * the last keys, reference fastmax_cuda_forward.cu:161-172; nq == 1 is one decoding step over
 * nk cached keys).  With nk > nq the library runs the keys every query sees and the square causal
 * part one after the other and merges them; fastmax_backward_saved does not cover that case. */
typedef struct FastmaxDesc {
  int32_t bh;        /* batch * heads */
  int32_t nq, nk;    /* query and key/value tokens */
  int32_t d;         /* head size, D == Dv; 32 or 64.  Also 128 for bf16 tensors on the _Float16 kernels (no
                        FASTMAX_FLAG_F32_COMPUTE, a0 > 0): dense tiles at any length (at that width the moment form
                        only pays beyond about D^2 keys), no normalisation fold, no causal nk > nq, no decoding state,
                        no FORCE_MOMENTS; anything else at 128 is FASTMAX_ERR_UNSUPPORTED */
  int32_t dtype;     /* FASTMAX_F32 or FASTMAX_BF16: element type of q,k,v,o,dO,dq,dk,dv */
  int32_t mask;
  int32_t p;         /* 1 or 2 */
  float a0, a1, a2;
  float inv_tau;
  int32_t chunk;     /* segment length of the causal moment scan; 0 = automatic */
  int32_t flags;
  FastmaxStrides sq, sk, sv, so, sg, sdo, sdq, sdk, sdv;   /* sg: strides of the fp32 denominator g (bh, n) */
  FastmaxNormFold norm;                                    /* all zero: off */
} FastmaxDesc;

/* Replaces the tensor allocations inside forward_cuda / backward_cuda
 * (reference fastmax_cuda_forward.cu:404-414, fastmax_cuda_backward.cu:563-571):
 * the caller owns all memory and asks here how much scratch a call needs. */
int fastmax_workspace_bytes(const FastmaxDesc* desc, size_t* forward_bytes, size_t* backward_bytes);

/* Replaces forward_cuda (reference fastmax_cuda.cpp:17-24 -> fastmax_cuda_forward.cu:366-456):
 * o (dtype) and the denominator g (fp32) for every query.  The reference returns both in one
 * (nq, bh, d+1) tensor; that layout is expressed by pointing g at column d of that tensor
 * with strides (d+1, bh*(d+1)).  workspace: >= forward_bytes, 256-byte aligned device memory. */
int fastmax_forward(const FastmaxDesc* desc, const void* q, const void* k, const void* v,
                    void* o, float* g, void* workspace, size_t workspace_bytes, void* hip_stream);

/* fastmax_forward for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose forward_cuda
 * allocates its output and four scratch tensors on every call (fastmax_cuda_forward.cu:404-414).
 * Same arguments, results and kernels as fastmax_forward, but the workspace is a buffer of
 * FASTMAX_STATIC_SCRATCH_BYTES that is part of the loaded library (one copy per GPU, held until the
 * process ends); the call allocates and frees nothing.  A problem whose forward_bytes
 * (fastmax_workspace_bytes) exceed that size is refused with FASTMAX_ERR_TOO_LARGE before anything is
 * launched.  All calls on one GPU share that GPU's buffer: calls that overlap in time on one GPU (two
 * streams, two threads) race and give wrong results; calls on one stream are ordered and safe.  The
 * buffer keeps the last call's contents; nothing in it needs clearing between calls.
 * FASTMAX_FLAG_SAVE_FOR_BACKWARD is honoured (the saved data then lives in the static buffer, until the
 * next call).  The first call on a device looks the buffer's address up and must not be made while a
 * stream capture is in progress; later calls may be captured. */
#define FASTMAX_STATIC_SCRATCH_BYTES (64u << 20)
int fastmax_forward_static(const FastmaxDesc* desc, const void* q, const void* k, const void* v,
                           void* o, float* g, void* hip_stream);

/* Replaces backward_cuda (reference fastmax_cuda.cpp:26-32 -> fastmax_cuda_backward.cu:518-613):
 * gradients of sum(o * dO) with respect to q, k and v, where s_ij = (q_i . k_j) * inv_tau.
 * o and g are the forward results.  d_o is not modified (the reference divides it by g in place,
 * fastmax_cuda_backward.cu:494-501). */
int fastmax_backward(const FastmaxDesc* desc, const void* q, const void* k, const void* v,
                     const void* o, const float* g, const void* d_o,
                     void* dq, void* dk, void* dv,
                     void* workspace, size_t workspace_bytes, void* hip_stream);

/* Same as fastmax_backward, reusing the workspace a forward call with FASTMAX_FLAG_SAVE_FOR_BACKWARD
 * left behind for the same desc, q, k, v (no counterpart in the reference, which recomputes
 * everything: fastmax_cuda_backward.cu:101-188 rebuilds the running key sums).  The key-side
 * conversions and the prefix-state build are skipped.  forward_workspace is only read. */
int fastmax_backward_saved(const FastmaxDesc* desc, const void* q, const void* k, const void* v,
                           const void* o, const float* g, const void* d_o,
                           void* dq, void* dk, void* dv,
                           const void* forward_workspace, size_t forward_workspace_bytes,
                           void* workspace, size_t workspace_bytes, void* hip_stream);

/* Incremental decoding on a persistent moment state (the running sums of fastmax_cuda_forward.cu:160-276
 * kept between calls; the reference's generation loop, transformer/eval.py:8-32, re-runs the whole context
 * for every new token).  The state of a batch*head is the fp32 sums over all keys so far of [1, k', k' x k']
 * times [v, 1] with k' = k * inv_tau, the symmetric order-2 part kept once per pair of features:
 * fastmax_decode_state_bytes(desc) bytes for desc->bh of them (0.70 MB per batch*head at d = 64, order 2;
 * 41 KB at order 1), whatever the number of keys.  The layout is the library's own (a state is only ever
 * passed back to these two calls).  A zero-filled buffer
 * is the empty state.  desc: bh, d, dtype, p, a0..a2, inv_tau and the strides named below are used; mask,
 * chunk, flags and norm are ignored (decoding is causal by construction and needs unnormalised q, k: the
 * max-norm depends on every token).
 *   fastmax_decode_absorb: adds desc->nk tokens (k, v: strides sk, sv) to the state, e.g. a prompt whose
 *     own outputs come from fastmax_forward.  One launch.  bf16 tensors at d = 64, order 2, 64 tokens or more:
 *     summed with matrix instructions on _Float16 operands (k', and the products v k'), fp32 sums (4 096 tokens
 *     at 16 batch*heads: 0.10 ms); otherwise token after token in fp32.
 *   fastmax_decode_step: adds one token (k, v) and reads the state out for its query q (strides sq; the
 *     query sees its own key, as in causal attention): o (strides so, one token) and g (sg).  scratch is
 *     not used any more (a step is one launch; the argument and fastmax_decode_scratch_bytes stay for
 *     callers built against the earlier signature; null is accepted).  desc->nq and nk are ignored (one token).
 * Both enqueue on the stream and allocate nothing; a step is one launch that reads and writes the state once. */
size_t fastmax_decode_state_bytes(const FastmaxDesc* desc);
size_t fastmax_decode_scratch_bytes(const FastmaxDesc* desc);
int fastmax_decode_absorb(const FastmaxDesc* desc, const void* k, const void* v, float* state, void* hip_stream);
int fastmax_decode_step(const FastmaxDesc* desc, const void* q, const void* k, const void* v, float* state,
                        void* o, float* g, float* scratch, void* hip_stream);

/* Fused normalisation pass over one (bh, n, d) tensor.  Replaces apply_rpe_and_temp, calc_norms,
 * find_max and apply_norm (reference fastmax_cuda_forward.cu:282-338) with the semantics the
 * Python variants define:
 *   y = scale * (x - centre) / max_n || x_n - centre ||_2     when max_norm != 0
 *   y = scale * (x - centre)                                   otherwise
 * centre: 0 none; 1 mean over the feature axis (fastattention_einops.py:327-334);
 *         2 mean over the token axis (score_function.py:42-47).
 * x and y may be the same buffer with the same strides.
 * stats: device scratch of fastmax_normalize_stats_bytes(desc) bytes (8-byte aligned), or null
 * when max_norm == 0 and centre != 2.  Every workgroup leaves its partial maximum / column sums
 * there and the next kernel joins them in a fixed order: no atomics, no clearing beforehand, the
 * same bits on every run. */
typedef struct FastmaxNormDesc {
  int32_t bh, n, d;
  int32_t dtype;
  int32_t centre;
  int32_t max_norm;
  float scale;
  FastmaxStrides sx, sy;
} FastmaxNormDesc;
size_t fastmax_normalize_stats_bytes(const FastmaxNormDesc* desc);
int fastmax_normalize(const FastmaxNormDesc* desc, const void* x, void* y, float* stats,
                      void* hip_stream);

/* Statistics for FastmaxNormFold: one read of x (desc->bh, n, d, dtype, sx are used), leaving
 * fastmax_maxnorm_stats_bytes(bh, n) bytes in `keys` (8-byte aligned device memory): per 256 tokens the
 * largest squared token norm and its token.  A second tensor of the same batch*heads, head size and type
 * (k beside q) can go in the same launch: desc1 / x1 / keys1, or null. */
size_t fastmax_maxnorm_stats_bytes(int32_t bh, int32_t n);
int fastmax_maxnorm_stats(const FastmaxNormDesc* desc0, const void* x0, void* keys0,
                          const FastmaxNormDesc* desc1, const void* x1, void* keys1, void* hip_stream);

/* Gradient of fastmax_normalize with respect to x, given dy (the gradient with respect to y).
 * The reference's extension has no counterpart: fastmax_cuda_backward.cu:518-613 returns the
 * gradients with respect to the already normalised q and k and the normalisation's own Jacobian
 * is dropped; its Python variants get it from autograd (score_function.py:40-55,
 * fastattention_einops.py:327-334), which this entry point reproduces:
 *   dx_n = (scale / m) * ( C(dy)_n - ([n == n*] - [centre == 2] / N) * (B / m^2) * c_{n*} )
 * with c = x - centre, m = max_n ||c_n|| reached at token n* (the first one among equal norms),
 * B = sum dy * c, and C(.) the same centring applied to dy; dx = scale * C(dy) when max_norm == 0.
 * desc->sx: strides of x and of dx; desc->sy: strides of dy.  dx may be the same buffer as dy
 * when their strides agree; it must not overlap x.
 * stats: device scratch of fastmax_normalize_backward_stats_bytes(desc) bytes (8-byte aligned),
 * or null when max_norm == 0 and centre != 2. */
size_t fastmax_normalize_backward_stats_bytes(const FastmaxNormDesc* desc);
int fastmax_normalize_backward(const FastmaxNormDesc* desc, const void* x, const void* dy, void* dx,
                               float* stats, void* hip_stream);

/* The two element-wise steps the reference's forward_cuda carries switched off, for callers that switch
 * them on.  desc: bh, n, d, dtype; sx: strides of the input (and of `noise`), sy: strides of the output,
 * which may be the input buffer itself when the strides agree.
 *
 * fastmax_key_rpe replaces the addition in apply_rpe_and_temp (reference fastmax_cuda_forward.cu:282-292,
 * commented out at :289):  k[l][m] = k[l][m] / tau + rpe[(l + n) % (2 n - 1)][m], rpe a contiguous fp32
 * (2 n - 1, d) table (rpe_matrix_creator, transformer/model.py:218-247).  The operator divides by tau in
 * its loads, so this writes k_out = k + temperature * rpe[..]; pass the result as k with the same inv_tau.
 * dk of the operator is then also the gradient with respect to the k given here.
 *
 * fastmax_output_noise replaces apply_dropout (fastmax_cuda_forward.cu:340-349, called with scale 0 at
 * :443):  o_out = o * (1 + scale * noise), noise of o's type and strides.  Applied to dO with the same
 * noise it is the step's backward. */
int fastmax_key_rpe(const FastmaxNormDesc* desc, const void* k, const float* rpe, void* k_out, float temperature,
                    void* hip_stream);
int fastmax_output_noise(const FastmaxNormDesc* desc, const void* o, const void* noise, void* o_out, float scale,
                         void* hip_stream);

const char* fastmax_status_string(int status);

/* Library version: major * 10000 + minor * 100 + patch. */
int fastmax_version(void);

/* Self-check of the matrix-core lane layout the kernels assume: runs one 32x32 MFMA tile per
 * element type on known operands and writes, for each of the 64 lanes and 16 accumulator
 * registers, the value found (out_f16 and out_f32: 1024 floats each, device memory). */
int fastmax_probe_mfma(float* out_f16, float* out_f32, void* hip_stream);

/* Self-check of the transposing LDS read (ds_read_b64_tr_b16) the _Float16 kernels use for transposed
 * fragments: one wavefront reads a 16 x 64 tile holding 64 * row + col; lane l addresses the four
 * values at (row l % 16, columns 4 * (l / 16) ..).  out: 256 floats (device memory), four per lane.
 * Expected: lane l, value t = 64 * (4 t + (l % 16) / 4) + 4 * (l / 16) + l % 4. */
int fastmax_probe_lds_transpose(float* out, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* FASTMAX_HIP_H_ */
