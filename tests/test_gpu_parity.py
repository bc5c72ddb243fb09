"""GPU parity tests: the HIP path through the C ABI against the CPU oracle on the
same seeded inputs.  Tolerances: rel-L2 1e-5 (fp32), 2e-2 (bf16, oracle fed the
bf16-rounded inputs)."""
import pytest
import torch

from tests.parity import (check_batch_head_strides, check_decode, check_forward, check_forward_backward,
                          check_norm_fold, make_inputs)
from reproducing_fastmax_results_amd._capi import FLAG_FORCE_DENSE, FLAG_FORCE_MOMENTS

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    from reproducing_fastmax_results_amd._capi import get_lib
    return get_lib()


@pytest.fixture(scope="module")
def bench_lib():
    """The bench build of the library (the product's sources with -DFM_BENCH_AIDS)."""
    from reproducing_fastmax_results_amd._capi import get_bench_lib
    return get_bench_lib()


DEV = "cuda:0"


def test_mfma_lane_layout(lib):
    """The kernels assume: lane l owns D[8*(e/4) + 4*(l/32) + e%4][l%32] of a 32x32 tile."""
    a16, a32 = lib.probe_mfma(DEV)
    torch.cuda.synchronize()
    lane = torch.arange(64).view(64, 1)
    e = torch.arange(16).view(1, 16)
    row = 8 * (e // 4) + 4 * (lane // 32) + e % 4
    col = lane % 32
    want = ((row + 1) * 100 + (col + 1)).float()
    assert torch.equal(a16.cpu(), want)
    assert torch.equal(a32.cpu(), want)


def test_matrix_rate_probe_runs(bench_lib):
    """The bench's yardstick: a register-only loop of matrix products; here only that it runs, writes
    every checksum and reports a rate (16 workgroups, 64 rounds)."""
    lib = bench_lib
    import ctypes as C
    out = torch.full((16 * 256,), float("nan"), device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.lib.fastmax_probe_mfma_rate(16, 64, C.c_void_p(out.data_ptr()), C.c_void_p(stream)) == 0
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    assert lib.mfma_rate(DEV, workgroups=256, iters=200) > 0.0


def test_lds_fed_mix_probe_runs(bench_lib):
    """The second yardstick (matrix products fed from LDS with the dense kernels' instruction mix): runs for one and
    two own tiles, writes every checksum, rejects anything else."""
    lib = bench_lib
    import ctypes as C
    stream = torch.cuda.current_stream().cuda_stream
    for tiles in (1, 2):
        out = torch.full((8 * 256,), float("nan"), device=DEV)
        assert lib.lib.fastmax_probe_mix_rate(8, 16, tiles, C.c_void_p(out.data_ptr()), C.c_void_p(stream)) == 0
        torch.cuda.synchronize()
        assert bool(torch.isfinite(out).all())
    out = torch.zeros(8 * 256, device=DEV)
    assert lib.lib.fastmax_probe_mix_rate(8, 16, 3, C.c_void_p(out.data_ptr()), C.c_void_p(stream)) != 0
    assert lib.lib.fastmax_probe_mix_rate(0, 16, 1, C.c_void_p(out.data_ptr()), C.c_void_p(stream)) != 0
    assert lib.lib.fastmax_probe_mix_rate(8, 16, 1, None, C.c_void_p(stream)) != 0
    assert lib.mix_rate(DEV, 1, iters=100) > 0.0


def test_bench_build_matches_the_product_and_times_its_kernels(lib, bench_lib):
    """The bench build runs the same kernels (bit-identical results) and its per-kernel events name them."""
    q, k, v, go = make_inputs(3, 700, 700, 64, torch.bfloat16, DEV, seed=5)
    kw = dict(mask=True, inv_tau=0.05, p=2)
    o0, g0 = lib.forward(q, k, v, **kw)
    bench_lib.profile_begin()
    o1, g1 = bench_lib.forward(q, k, v, **kw)
    recs = bench_lib.profile_end()
    assert torch.equal(o0, o1) and torch.equal(g0, g1)
    assert {"transpose", "fwd"} <= {name for name, _ in recs} and all(ms > 0.0 for _, ms in recs)
    assert not hasattr(lib.lib, "fastmax_profile_begin")      # the product library carries no bench aid


def test_lds_transpose_read_layout(lib):
    """The kernels (and the host simulator) assume: inside each group of 16 lanes, lane i receives
    element i % 4 of the four-value words addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4."""
    got = lib.probe_lds_transpose(DEV)
    torch.cuda.synchronize()
    lane = torch.arange(64).view(64, 1)
    t = torch.arange(4).view(1, 4)
    want = (64 * (4 * t + (lane % 16) // 4) + 4 * (lane // 16) + lane % 4).float()
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("d", [32, 64])
def test_forward_dense_small(lib, dtype, mask, p, d):
    print(f"case dense dtype={dtype} mask={mask} p={p} d={d}", flush=True)
    check_forward(lib, 3, 333, d, dtype, DEV, mask=mask, p=p, flags=FLAG_FORCE_DENSE, seed=1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("d", [32, 64])
def test_forward_moments_small(lib, dtype, mask, p, d):
    print(f"case moments dtype={dtype} mask={mask} p={p} d={d}", flush=True)
    check_forward(lib, 3, 1100, d, dtype, DEV, mask=mask, p=p, chunk=256, flags=FLAG_FORCE_MOMENTS, seed=2)


def test_forward_config1(lib):
    # Fastmax order-2 forward, unmasked, fp32: B=1, H=2, N=256, D=Dv=32
    for flags in (FLAG_FORCE_DENSE, FLAG_FORCE_MOMENTS):
        print(f"case config1 flags={flags}", flush=True)
        check_forward(lib, 2, 256, 32, torch.float32, DEV, mask=False, p=2, flags=flags, seed=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk", [0, 1024, 2048])
def test_forward_config2_heads(lib, dtype, chunk):
    # causal order 2, N=4096, D=64: 4 of the 32 (b, h) slices against the fp64 closed form;
    # chunk 0 is the library's own choice (one segment at this length), the others go through the states
    print(f"case config2 fwd dtype={dtype} chunk={chunk}", flush=True)
    check_forward(lib, 4, 4096, 64, dtype, DEV, mask=True, p=2, seed=1, chunk=chunk)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_forward_ragged_and_cross(lib, dtype):
    print(f"case ragged dtype={dtype}", flush=True)
    check_forward(lib, 2, 1, 64, dtype, DEV, mask=True, p=2, seed=3)
    check_forward(lib, 2, 50, 32, dtype, DEV, mask=False, p=2, seed=4)          # ViT shape: 49 patches + CLS
    check_forward(lib, 2, 257, 64, dtype, DEV, mask=False, p=2, nk=513, seed=5)  # nq != nk, unmasked
    check_forward(lib, 1, 700, 64, dtype, DEV, mask=False, p=2, nk=4500, seed=6)  # automatic moment path


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("d", [32, 64])
def test_backward_dense_small(lib, dtype, mask, p, d):
    print(f"case bwd dense dtype={dtype} mask={mask} p={p} d={d}", flush=True)
    check_forward_backward(lib, 3, 333, d, dtype, DEV, mask=mask, p=p, flags=FLAG_FORCE_DENSE, seed=7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("d", [32, 64])
def test_backward_moments_small(lib, dtype, mask, p, d):
    print(f"case bwd moments dtype={dtype} mask={mask} p={p} d={d}", flush=True)
    check_forward_backward(lib, 3, 1100, d, dtype, DEV, mask=mask, p=p, chunk=256, flags=FLAG_FORCE_MOMENTS, seed=8)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk", [0, 1024, 2048])
def test_backward_config2_heads(lib, dtype, chunk):
    # Fastmax order-2 causal forward and backward, N=4096, D=64 (4 of the 32 slices, fp64 closed form)
    print(f"case config2 fwd+bwd dtype={dtype} chunk={chunk}", flush=True)
    check_forward_backward(lib, 4, 4096, 64, dtype, DEV, mask=True, p=2, seed=9, chunk=chunk)
    check_forward_backward(lib, 4, 4096, 64, dtype, DEV, mask=True, p=2, seed=9, chunk=chunk, saved=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_sequence_default_segments(lib, dtype):
    # beyond 6144 tokens the library cuts the sequence into 1024-token segments on its own
    print(f"case long dtype={dtype}", flush=True)
    check_forward_backward(lib, 1, 7000, 64, dtype, DEV, mask=True, p=2, seed=21, saved=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d", [32, 64])
def test_order1_default_segments(lib, dtype, d):
    # order 1 beyond 1024 tokens: 256-token segments summed apart, then scanned (16 and 28 segments, the
    # second with a ragged end); unmasked with many keys: one total over all keys by a single walk step
    print(f"case order1 segments dtype={dtype} d={d}", flush=True)
    check_forward_backward(lib, 3, 4096, d, dtype, DEV, mask=True, p=1, seed=22, saved=True)
    check_forward_backward(lib, 2, 7000, d, dtype, DEV, mask=True, p=1, seed=23)
    check_forward_backward(lib, 2, 300, d, dtype, DEV, mask=False, p=1, nk=5000, seed=24)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_order2_states_mid_sized_batch(lib, dtype):
    # 16 <= batch*heads < 32 at D = 64: the state walk is serial over segments with one workgroup per CU
    print(f"case order2 mid batch dtype={dtype}", flush=True)
    check_forward_backward(lib, 16, 1100, 64, dtype, DEV, mask=True, p=2, chunk=256, seed=25)
    check_forward_backward(lib, 20, 1100, 64, dtype, DEV, mask=True, p=2, chunk=256, seed=26, saved=True)
    check_forward_backward(lib, 17, 300, 64, dtype, DEV, mask=False, p=2, nk=700, seed=27, flags=FLAG_FORCE_MOMENTS)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_backward_ragged_and_cross(lib, dtype):
    print(f"case bwd ragged dtype={dtype}", flush=True)
    check_forward_backward(lib, 2, 1, 64, dtype, DEV, mask=True, p=2, seed=10)
    check_forward_backward(lib, 2, 50, 32, dtype, DEV, mask=False, p=2, seed=11)
    check_forward_backward(lib, 2, 257, 64, dtype, DEV, mask=False, p=2, nk=513, seed=12)
    check_forward_backward(lib, 1, 700, 64, dtype, DEV, mask=False, p=2, nk=4500, seed=13)
    check_forward_backward(lib, 1, 2500, 64, dtype, DEV, mask=True, p=2, seed=14, chunk=1024)   # ragged last segment
    check_forward_backward(lib, 2, 777, 32, dtype, DEV, mask=True, p=2, a=(1.0, 1.166666, 0.145833), tau_mult=1.0,
                           seed=15)                                                    # fitted (non-Taylor) coefficients


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d,bh", [(64, 32), (32, 64)])
def test_many_heads(lib, dtype, d, bh):
    # the head count of the benchmark (B*H = 32 at D = 64): exercises the XCD-aware
    # workgroup mapping (B*H a multiple of 8) and grids larger than the GPU
    print(f"case many heads dtype={dtype} d={d} bh={bh}", flush=True)
    check_forward_backward(lib, bh, 1100, d, dtype, DEV, mask=True, p=2, chunk=256, seed=16)
    check_forward_backward(lib, bh, 600, d, dtype, DEV, mask=False, p=2, flags=FLAG_FORCE_MOMENTS, seed=17)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
def test_backward_on_saved_forward_workspace(lib, dtype, mask, p):
    # fastmax_backward_saved: key-side copies and the prefix state come from the forward
    print(f"case saved dtype={dtype} mask={mask} p={p}", flush=True)
    check_forward_backward(lib, 8, 1100, 64, dtype, DEV, mask=mask, p=p, chunk=256, flags=FLAG_FORCE_MOMENTS,
                           seed=18, saved=True)
    check_forward_backward(lib, 3, 333, 32, dtype, DEV, mask=mask, p=p, flags=FLAG_FORCE_DENSE, seed=19, saved=True)
    check_forward_backward(lib, 2, 2500, 64, dtype, DEV, mask=mask, p=p, seed=20, saved=True, chunk=1024)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask,chunk", [(True, 0), (True, 256), (False, 0)])
def test_batch_and_head_strides(lib, dtype, mask, chunk):
    print(f"case two-level strides dtype={dtype} mask={mask} chunk={chunk}", flush=True)
    check_batch_head_strides(lib, 3, 4, 700, 64, dtype, DEV, mask=mask, p=2, chunk=chunk, seed=30)
    check_batch_head_strides(lib, 2, 8, 130, 32, dtype, DEV, mask=mask, p=1, chunk=chunk, seed=31)
    check_batch_head_strides(lib, 2, 4, 1300, 64, dtype, DEV, mask=mask, p=1, chunk=chunk, seed=32)   # order-1 segments
    check_batch_head_strides(lib, 5, 1, 300, 64, dtype, DEV, mask=mask, p=2, chunk=chunk, seed=33)    # one head per batch


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("nq,nk", [(1, 700), (300, 301), (513, 2100), (2048, 6000)])
def test_causal_more_keys_than_queries(lib, dtype, p, nq, nk):
    """Causal with nk > nq, queries aligned to the last keys (fastmax_cuda_forward.cu:161-172):
    prompt keys every query sees plus the square causal part (nq = 1: one decoding step)."""
    print(f"case causal nk>nq dtype={dtype} p={p} nq={nq} nk={nk}", flush=True)
    d = 64 if nq != 300 else 32
    check_forward_backward(lib, 3, nq, d, dtype, DEV, mask=True, p=p, nk=nk, seed=50)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("jacobian", [True, False])
def test_normalisation_folded_into_the_loads(lib, dtype, jacobian):
    """lim * x / max-norm of q and k applied as the kernels load the rows (one statistics pass, one read of q and
    k); gradients with respect to the raw tensors (fp64 autograd through the normalisation) or, like the
    reference's extension, with respect to the normalised ones."""
    print(f"case folded normalisation dtype={dtype} jacobian={jacobian}", flush=True)
    for p, chunk in ((2, 0), (2, 256), (1, 0), (1, 256)):
        check_norm_fold(lib, 3, 1100, 64, dtype, DEV, mask=True, p=p, chunk=chunk, seed=70 + p, jacobian=jacobian)
        check_norm_fold(lib, 2, 700, 32, dtype, DEV, mask=True, p=p, chunk=chunk, seed=72 + p, jacobian=jacobian, saved=False)
    check_norm_fold(lib, 2, 300, 64, dtype, DEV, mask=False, p=2, nk=700, seed=75, jacobian=jacobian, saved=False)
    check_norm_fold(lib, 2, 50, 32, dtype, DEV, mask=False, p=2, seed=76, jacobian=jacobian)
    check_norm_fold(lib, 8, 4096, 64, dtype, DEV, mask=True, p=2, seed=77, jacobian=jacobian, lim=1.0, tau=1.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("d", [32, 64])
def test_incremental_decoding_on_the_moment_state(lib, dtype, p, d):
    """fastmax_decode_absorb / fastmax_decode_step: a prompt absorbed into the persistent state, then one step per
    token, every step against the fp64 closed form of causal attention over the whole sequence; also decoding
    from the empty state, the reference's own test temperature, and the cached-keys route on the same tokens."""
    print(f"case decode state dtype={dtype} p={p} d={d}", flush=True)
    check_decode(lib, 6, 700, 640, d, dtype, DEV, p=p, seed=90)
    check_decode(lib, 4, 48, 0, d, dtype, DEV, p=p, seed=91, tau_mult=1.0)
    check_decode(lib, 4, 300, 290, d, dtype, DEV, p=p, seed=92, four_d=True)

    # one step against the library's own route over cached keys (causal, one query, all keys)
    import math
    from tests.parity import make_inputs, rel_err, TOL
    q, k, v, _ = make_inputs(3, 513, 513, d, dtype, DEV, seed=93)
    kw = dict(inv_tau=1.0 / (8.0 * math.sqrt(d)), p=p)
    state = lib.decode_state(k, **kw)
    lib.decode_absorb(k[:, :512], v[:, :512], state, **kw)
    o, g = lib.decode_step(q[:, 512:], k[:, 512:], v[:, 512:], state, **kw)
    o2, g2 = lib.forward(q[:, 512:].contiguous(), k, v, mask=True, **kw)
    assert rel_err(o, o2) < TOL[dtype] and rel_err(g, g2) < TOL[dtype]


@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("mask", [True, False])
def test_heads_of_128(lib, p, mask):
    """bf16 tensors at D = 128 (dense tiles only): forward and backward, saved and not, ragged lengths, unequal nq and
    nk without a mask, a sequence long enough that D = 64 would use states, and the statuses of what it leaves out."""
    print(f"case heads of 128 p={p} mask={mask}", flush=True)
    check_forward_backward(lib, 3, 300, 128, torch.bfloat16, DEV, mask=mask, p=p, seed=120, saved=True)
    check_forward_backward(lib, 2, 1000, 128, torch.bfloat16, DEV, mask=mask, p=p, seed=121, saved=False, tau_mult=1.0)
    check_forward_backward(lib, 8, 2048, 128, torch.bfloat16, DEV, mask=mask, p=p, seed=122, saved=True)
    if not mask:
        check_forward_backward(lib, 2, 130, 128, torch.bfloat16, DEV, mask=False, p=p, nk=517, seed=123, saved=True)
    else:
        check_forward_backward(lib, 1, 8200, 128, torch.bfloat16, DEV, mask=True, p=p, seed=124, saved=True)
        check_batch_head_strides(lib, 2, 3, 260, 128, torch.bfloat16, DEV, mask=True, p=p, seed=125)
    from reproducing_fastmax_results_amd._capi import FastmaxError
    q, k, v, go = (torch.randn(2, 64, 128, device=DEV) for _ in range(4))
    with pytest.raises(FastmaxError):
        lib.forward(q, k, v, mask=mask, inv_tau=0.1, p=p)                # fp32 tensors


def test_prompt_absorbed_with_matrix_instructions(lib):
    """bf16 tensors, D = 64, order 2: prompts of 64 tokens and more are summed by k_decode_absorb_mma.  Decoding after
    a long prompt against the causal closed form; the state against the one k_decode builds from the same tokens in
    pieces below the threshold (operands rounded to _Float16: 5e-3 per entry, 1e-4 over the state); absorbing in two
    calls (into a state that is not empty, strided (b, h, n, d) views) against one call."""
    import math
    from tests.parity import check_decode, make_inputs
    print("case absorb mma: decode after a 4000-token prompt", flush=True)
    check_decode(lib, 2, 4008, 4000, 64, torch.bfloat16, DEV, p=2, seed=95)
    check_decode(lib, 4, 203, 199, 64, torch.bfloat16, DEV, p=2, seed=96, four_d=True)
    bh, n, d = 16, 2500, 64
    q, k, v, _ = make_inputs(bh, n, n, d, torch.bfloat16, DEV, 7)
    kw = dict(inv_tau=1.0 / (8.0 * math.sqrt(d)), p=2, a0=1.0, a1=1.0, a2=0.5)
    one, two, small = (lib.decode_state(k, **kw) for _ in range(3))
    print("case absorb mma: one call, two calls, pieces of 48", flush=True)
    lib.decode_absorb(k, v, one, **kw)
    lib.decode_absorb(k[:, :1000], v[:, :1000], two, **kw)
    lib.decode_absorb(k[:, 1000:], v[:, 1000:], two, **kw)
    for t0 in range(0, n, 48):
        lib.decode_absorb(k[:, t0:t0 + 48], v[:, t0:t0 + 48], small, **kw)
    torch.cuda.synchronize()
    assert float((one - two).norm() / one.norm()) < 1e-6
    assert float((one - small).norm() / small.norm()) < 1e-4
    live = small.abs() > 1e-3 * small.abs().max()
    assert float(((one - small).abs() / small.abs().clamp_min(1e-30))[live].max()) < 5e-3



@pytest.mark.parametrize("go_scale", [1e-7, 1e-4, 3e4])
def test_upstream_gradient_of_any_size(lib, go_scale):
    """Gradients are linear in dO, whose size is the caller's: a loss averaged over 16 x 1024 tokens hands over
    dO near 1e-6.  The bf16 path brings dO / g of every batch*head into the _Float16 range and back."""
    print(f"case upstream gradient size {go_scale}", flush=True)
    for p, chunk in ((2, 0), (2, 256), (1, 0), (1, 256)):
        check_forward_backward(lib, 4, 1024, 64, torch.bfloat16, DEV, mask=True, p=p, chunk=chunk, seed=61,
                               go_scale=go_scale, saved=True)
    # order 1 beyond 1024 tokens runs on 128-token segments summed in runs, with a scale of its own
    for n in (1100, 4096):
        check_forward_backward(lib, 4, n, 64, torch.bfloat16, DEV, mask=True, p=1, seed=64, go_scale=go_scale, saved=True)
    check_forward_backward(lib, 2, 300, 32, torch.bfloat16, DEV, mask=False, p=2, nk=700, seed=62, go_scale=go_scale)
    check_forward_backward(lib, 2, 513, 64, torch.bfloat16, DEV, mask=True, p=2, nk=2100, seed=63, go_scale=go_scale)


@pytest.mark.parametrize("chunk", [0, 512])
def test_values_with_a_common_component(lib, chunk):
    """Tokens of a trained layer share a large common component (here: token-mean 0.7 of an rms of 1).  Then o_i is
    close to every v_j, gh.v_j and c_i = gh.o_i are of one size, and dS = f'(s)(gh.v - c) is their small difference:
    an error in c has one sign along a whole row of keys and adds up in sum_j dk_j, which is what the weight
    gradient of the key projection sees.  The backward on a kept forward workspace reads what bf16 rounding took
    from o there and keeps c in fp32: dq, dk, dv within the bar, and the sums over tokens (rel-L2 per slice of the
    (bh, d) sums) within three times what rounding the exact gradients to bf16 does to those sums, where the backward
    that only has the caller's bf16 o is several times further off."""
    import math
    from tests.parity import TOL, oracle_all, rel_err
    print(f"case common component chunk={chunk}", flush=True)
    bh, n, d = 4, 2048, 64
    gen = torch.Generator().manual_seed(44)
    q, k, v = ((0.7 * torch.randn(bh, n, d, generator=gen) + 0.7 * torch.randn(bh, 1, d, generator=gen)).bfloat16().to(DEV)
               for _ in range(3))
    go = torch.randn(bh, n, d, generator=gen).bfloat16().to(DEV)
    tau = 8.0 * math.sqrt(d)
    kw = dict(mask=True, inv_tau=1.0 / tau, p=2, chunk=chunk)
    o, g, ws = lib.forward(q, k, v, save=True, **kw)
    saved = lib.backward(q, k, v, o, g, go, saved=ws, **kw)
    plain = lib.backward(q, k, v, o, g, go, **kw)
    ref = oracle_all(q, k, v, go, mask=True, tau=tau, p=2)
    tol = TOL[torch.bfloat16]
    for name, x, r in zip(("dq", "dk", "dv"), saved, ref[2:]):
        assert rel_err(x, r) < tol, f"{name} rel-L2 {rel_err(x, r):.3e}"
    sums = {name: rel_err(x.double().sum(1), r.sum(1)) for name, x, r in zip(("dq", "dk", "dv"), saved, ref[2:])}
    sums_plain = {name: rel_err(x.double().sum(1), r.sum(1)) for name, x, r in zip(("dq", "dk", "dv"), plain, ref[2:])}
    floor = {name: rel_err(r.bfloat16().double().sum(1), r.sum(1)) for name, r in zip(("dq", "dk", "dv"), ref[2:])}
    print(f"  token sums, kept workspace {sums}, caller's o only {sums_plain}, bf16-rounded exact gradients {floor}", flush=True)
    for name in sums:
        assert sums[name] < 4.0 * floor[name] + 1e-3, (name, sums, floor)
    assert sums["dk"] < 0.5 * sums_plain["dk"], (sums, sums_plain)


@pytest.mark.parametrize("n,p,chunk", [(700, 2, 0), (2048, 2, 512), (2048, 1, 0)])
def test_bf16_value_range(lib, n, p, chunk):
    """The range of v that include/fastmax_hip.h states for bf16 tensors: entries of 1e-4 .. 1e2 in magnitude meet
    the bar on every tensor (one segment, order-2 states, the order-1 path of long sequences); beyond it (1e3, 1e4) a
    result is within the bar or not finite, never finite and wrong; FASTMAX_FLAG_F32_COMPUTE meets the bar there."""
    import math
    from reproducing_fastmax_results_amd._capi import FLAG_F32_COMPUTE
    from tests.parity import TOL, oracle_all, rel_err
    bh, d, tol = 2, 64, TOL[torch.bfloat16]
    tau = 8.0 * math.sqrt(d)

    def run(vs, flags=0):
        gen = torch.Generator().manual_seed(3)
        q, k = (torch.randn(bh, n, d, generator=gen).bfloat16() for _ in range(2))
        v = (vs * torch.randn(bh, n, d, generator=gen)).bfloat16()
        go = torch.randn(bh, n, d, generator=gen).bfloat16()
        kw = dict(mask=True, inv_tau=1.0 / tau, p=p, chunk=chunk, flags=flags)
        qd, kd, vd, gd = (t.to(DEV) for t in (q, k, v, go))
        if flags:
            o, g = lib.forward(qd, kd, vd, **kw)
            grads = lib.backward(qd, kd, vd, o, g, gd, **kw)
        else:
            o, g, ws = lib.forward(qd, kd, vd, save=True, **kw)
            grads = lib.backward(qd, kd, vd, o, g, gd, saved=ws, **kw)
        ref = oracle_all(q, k, v, go, mask=True, tau=tau, p=p)
        return list(zip(("o", "g", "dq", "dk", "dv"), (o, g) + tuple(grads), ref))

    for vs in (1e-4, 1e-2, 1e2):
        print(f"case bf16 value range n={n} p={p} chunk={chunk} v x {vs:g}", flush=True)
        for name, x, r in run(vs):
            assert bool(torch.isfinite(x).all()) and rel_err(x, r) < tol, f"{name} at v x {vs:g}: {rel_err(x, r):.3e}"
    for vs in (1e3, 1e4):
        print(f"case bf16 value range n={n} p={p} chunk={chunk} v x {vs:g} (beyond)", flush=True)
        for name, x, r in run(vs):
            assert (not bool(torch.isfinite(x).all())) or rel_err(x, r) < tol, f"{name} finite but wrong at v x {vs:g}"
        for name, x, r in run(vs, FLAG_F32_COMPUTE):
            assert bool(torch.isfinite(x).all()) and rel_err(x, r) < tol, f"{name} in fp32 at v x {vs:g}"


def test_bf16_range_is_loud_not_wrong(lib):
    """bf16 tensors are computed in _Float16.  Inside the documented range (|s| <= 250) the results meet
    the bf16 bar; beyond it a result is either still within the bar or not finite, never a finite wrong
    number; FASTMAX_FLAG_F32_COMPUTE meets the bar on the same inputs.  Also a0 = 0 (denominators that do
    not grow with the token index)."""
    import math
    from oracle import fastmax_oracle as O
    from reproducing_fastmax_results_amd._capi import FLAG_F32_COMPUTE
    from tests.parity import TOL, make_inputs, oracle_all, rel_err
    bh, n, d = 2, 700, 64
    tol = TOL[torch.bfloat16]

    def run(scale, flags, a, tau):
        q, k, v, go = make_inputs(bh, n, n, d, torch.bfloat16, DEV, seed=60, scale=scale)
        kw = dict(mask=True, inv_tau=1.0 / tau, a0=a[0], a1=a[1], a2=a[2], p=2, flags=flags)
        o, g = lib.forward(q, k, v, **kw)
        grads = lib.backward(q, k, v, o, g, go, **kw)
        ref = oracle_all(q, k, v, go, mask=True, tau=tau, p=2, a=a)
        smax = float((q.double() @ k.double().transpose(1, 2)).abs().max()) / tau
        return smax, list(zip((o, g) + tuple(grads), ref))

    taylor, tau = (1.0, 1.0, 0.5), 8.0 * math.sqrt(d)
    smax, pairs = run(15.0, 0, taylor, tau)                        # the edge of the documented range
    print(f"case bf16 range smax={smax:.0f}", flush=True)
    assert 120.0 < smax <= 250.0
    for x, r in pairs:
        assert bool(torch.isfinite(x).all()) and rel_err(x, r) < tol
    for scale in (30.0, 300.0):
        smax, pairs = run(scale, 0, taylor, tau)
        print(f"case bf16 range scale={scale} smax={smax:.0f}", flush=True)
        for x, r in pairs:
            assert (not bool(torch.isfinite(x).all())) or rel_err(x, r) < tol, f"finite but wrong at scale {scale}"
        _, pairs = run(scale, FLAG_F32_COMPUTE, taylor, tau)
        for x, r in pairs:
            assert bool(torch.isfinite(x).all()) and rel_err(x, r) < tol
    # a0 = 0: the weights change sign around s = 0 and the sums cancel (some |g_i| are a thousandth of the sum
    # of |f|); the library computes such problems in fp32 by itself
    for tau in (math.sqrt(d), 8.0 * math.sqrt(d)):
        _, pairs = run(1.0, 0, (0.0, 1.0, 0.5), tau)
        for x, r in pairs:
            assert bool(torch.isfinite(x).all()) and rel_err(x, r) < tol


def test_step_replays_as_a_hip_graph(lib):
    """The entry points allocate nothing and never synchronise, so a caller can capture forward and
    backward into one HIP graph.  Every replay (with eager work and synchronisations in between, and
    new input values in the captured buffers) must give what the eager call gives."""
    import math
    bh, n, d = 6, 1500, 64
    gen = torch.Generator().manual_seed(80)
    bufs = [torch.randn(bh, n, d, generator=gen).bfloat16().to(DEV) for _ in range(4)]
    q, k, v, go = bufs
    kw = dict(mask=True, inv_tau=1.0 / (8.0 * math.sqrt(d)), p=2)

    def step():
        o, g, saved = lib.forward(q, k, v, save=True, **kw)
        return (o,) + tuple(lib.backward(q, k, v, o, g, go, saved=saved, **kw))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for rep in range(4):
        for b in bufs:                                   # new values in the captured input buffers
            b.copy_(torch.randn(bh, n, d, generator=gen).bfloat16())
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()                                    # eager, same inputs
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), f"replay {rep} differs from the eager call"


def _random_cases(count, seed):
    import random
    rng = random.Random(seed)
    cases = []
    for _ in range(count):
        d = rng.choice((32, 64))
        mask = rng.random() < 0.6
        nq = rng.choice((1, 2, 31, 33, 64, 127, 129, 255, 257, 300, 511, 640, 777, 1025, 1500))
        if mask:
            nk = nq if rng.random() < 0.7 else nq + rng.choice((1, 17, 128, 300))
        else:
            nk = rng.choice((5, 64, 130, 257, 900))     # one key makes dq = dk = 0 exactly: nothing to compare rounding noise with
        cases.append(dict(bh=rng.choice((1, 2, 3, 5)), nq=nq, nk=nk, d=d, mask=mask, p=rng.choice((1, 2)),
                          chunk=rng.choice((0, 0, 256)), dtype=rng.choice((torch.float32, torch.bfloat16)),
                          saved=mask and nk == nq and rng.random() < 0.5, seed=rng.randrange(1 << 20)))
    return cases


@pytest.mark.parametrize("case", _random_cases(48, 2024), ids=lambda c: "-".join(
    f"{k}{v}" for k, v in c.items() if k not in ("seed", "dtype")) + ("-bf16" if c["dtype"] == torch.bfloat16 else "-f32"))
def test_seeded_random_shapes(lib, case):
    """Forward and backward against the oracle on a fixed list of odd shapes (ragged lengths around
    the 32 / 64 / 128 / 256 tile sizes, cross attention, cached keys, both orders, segments)."""
    print(f"case random {case}", flush=True)
    check_forward_backward(lib, case["bh"], case["nq"], case["d"], case["dtype"], DEV, mask=case["mask"], p=case["p"],
                           nk=case["nk"], chunk=case["chunk"], seed=case["seed"], saved=case["saved"])

