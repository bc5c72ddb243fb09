"""GPU parity at the full benchmark sizes, every (b, h) slice, through checks whose cost does
not grow with the square of the sequence length:

* the upstream gradient is zero outside a few query rows, so only those rows of the score
  matrix enter any result and the fp64 closed form restricted to them
  (``oracle.sampled_rows_forward_backward``) is an exact oracle for o and g at the rows, dq
  everywhere (zero off the rows) and the whole of dk and dv;
* ``a1 = a2 = 0`` turns causal Fastmax into the running mean of v (every row, fp64 cumsum);
* keys and values after a token do not reach it: the outputs of the first tokens are the
  bits of a run on the truncated sequence.

Tolerances as everywhere: rel-L2 1e-5 (fp32), 2e-2 (bf16, oracle fed the rounded inputs)."""
import math

import pytest
import torch

from oracle import fastmax_oracle as O
from tests.parity import TOL, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def lib():
    from reproducing_fastmax_results_amd._capi import get_lib
    return get_lib()


def _inputs(bh, n, d, dtype, seed, scale):
    gen = torch.Generator().manual_seed(seed)
    return [(s * torch.randn(bh, n, d, generator=gen)).to(dtype) for s in (scale, scale, scale, 1.0)]


def _rows(n, count, seed, seg):
    """first and last token, both sides of the 256-, 1024- and 2048-token segment boundaries
    and of a 128-token block, seeded random rows, and one seeded random row inside EVERY stretch of
    ``seg`` tokens: with ``seg`` the segment length of the moment scan every segment holds a query with
    an upstream gradient, so every segment's prefix state (o, dq) and suffix state (dk, dv of all earlier
    keys) enters the compared results"""
    fixed = [0, 1, 31, 32, 127, 128, 255, 256, 1023, 1024, 2047, 2048, n // 2 - 1, n // 2, n - 2, n - 1]
    gen = torch.Generator().manual_seed(seed)
    rnd = torch.randint(0, n, (count,), generator=gen).tolist()
    nseg = (n + seg - 1) // seg
    inside = torch.randint(0, seg, (nseg,), generator=gen)
    per_seg = [min(i * seg + int(inside[i]), n - 1) for i in range(nseg)]
    rows = torch.tensor(sorted({r for r in fixed + rnd + per_seg if 0 <= r < n}))
    assert len(set((rows // seg).tolist())) == nseg
    return rows


def _check_sparse_rows(lib, bh, n, d, dtype, p, seed, scale, chunk=0, count=48, seg=256, tau_mult=8.0):
    q, k, v, go = _inputs(bh, n, d, dtype, seed, scale)
    rows = _rows(n, count, seed + 1, seg)
    sparse = torch.zeros_like(go)
    sparse[:, rows] = go[:, rows]
    tau = tau_mult * math.sqrt(d)
    kw = dict(mask=True, inv_tau=1.0 / tau, p=p, chunk=chunk)
    qd, kd, vd, gd = (t.to(DEV) for t in (q, k, v, sparse))
    o, g, ws = lib.forward(qd, kd, vd, save=True, **kw)
    dq, dk, dv = lib.backward(qd, kd, vd, o, g, gd, saved=ws, **kw)
    torch.cuda.synchronize()
    ref = O.sampled_rows_forward_backward(q, k, v, rows, go[:, rows], tau=tau, p=p)
    dq = dq.cpu()
    off = torch.ones(n, dtype=torch.bool)
    off[rows] = False
    assert float(dq[:, off].float().abs().max()) == 0.0, "dq of a row without upstream gradient"
    got = (o.cpu()[:, rows], g.cpu()[:, rows], dq[:, rows], dk.cpu(), dv.cpu())
    names = ("o", "g", "dq", "dk", "dv")
    errs = {name: rel_err(x, r) for name, x, r in zip(names, got, ref)}
    for name, e in errs.items():
        assert e < TOL[dtype], f"{name} rel-L2 {e:.3e} (all: {errs})"
    # per slice as well: one bad (b, h) must not hide among the others
    for i in range(bh):
        for name, x, r in zip(names, got, ref):
            e = rel_err(x[i], r[i])
            assert e < TOL[dtype], f"slice {i}: {name} rel-L2 {e:.3e}"
    # dk and dv per stretch of ``seg`` keys and slice: one wrong suffix state must not hide in a sum over
    # the whole sequence.  Keys behind the last row with upstream gradient have dk = dv = 0 exactly, on both sides.
    worst = {}
    for name, x, r in (("dk", got[3], ref[3]), ("dv", got[4], ref[4])):
        x = _by_segment(x.double(), seg); r = _by_segment(r.double(), seg)
        num = (x - r).flatten(2).norm(dim=2); den = r.flatten(2).norm(dim=2)
        assert bool((num[den == 0] == 0).all()), f"{name}: non-zero where the reference is exactly zero"
        e = (num / den.clamp_min(1e-300))[den > 0]
        worst[name] = float(e.max())
        assert worst[name] < TOL[dtype], f"{name}: worst rel-L2 over {seg}-key stretches {worst[name]:.3e}"
    print(f"  errs {errs} worst per stretch {worst}", flush=True)
    return errs


def _by_segment(x, seg):
    """(bh, n, d) -> (bh, ceil(n / seg), seg, d), zero padded"""
    bh, n, d = x.shape
    pad = (-n) % seg
    if pad:
        x = torch.cat([x, x.new_zeros(bh, pad, d)], dim=1)
    return x.view(bh, -1, seg, d)


def _check_running_mean(lib, bh, n, d, dtype, p, seed, chunk=0):
    q, k, v, _ = _inputs(bh, n, d, dtype, seed, 1.0)
    o, g = lib.forward(q.to(DEV), k.to(DEV), v.to(DEV), mask=True, inv_tau=1.0 / (8.0 * math.sqrt(d)),
                       a0=1.0, a1=0.0, a2=0.0, p=p, chunk=chunk)
    count = torch.arange(1, n + 1, dtype=torch.float64)
    want = v.double().cumsum(1) / count.view(1, n, 1)
    assert torch.equal(g.cpu().double(), count.expand(bh, n)), "g must be the number of visible keys"
    e = rel_err(o, want)
    assert e < TOL[dtype], f"o rel-L2 {e:.3e}"


def _prefix_runs(lib, bh, n, cut, d, dtype, p, seed, scale, chunk):
    """forward on the whole sequence and on its first ``cut`` tokens, same segment length (so the
    same sums in the same order)"""
    q, k, v, _ = _inputs(bh, n, d, dtype, seed, scale)
    kw = dict(mask=True, inv_tau=1.0 / (8.0 * math.sqrt(d)), p=p, chunk=chunk)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    o, g = lib.forward(qd, kd, vd, **kw)
    o2, g2 = lib.forward(qd[:, :cut].contiguous(), kd[:, :cut].contiguous(), vd[:, :cut].contiguous(), **kw)
    torch.cuda.synchronize()
    return o, g, o2, g2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_config2_all_slices(lib, dtype):
    # causal order 2, B*H = 32, N = 4096, D = 64: all 32 slices
    print(f"case full config2 dtype={dtype}", flush=True)
    _check_sparse_rows(lib, 32, 4096, 64, dtype, 2, seed=101, scale=1.0)
    _check_running_mean(lib, 32, 4096, 64, dtype, 2, seed=102)


@pytest.mark.parametrize("chunk", [1024, 2048])
def test_config2_all_slices_through_states(lib, chunk):
    # the same shape cut into segments, through their prefix / suffix states
    print(f"case full config2 chunk={chunk}", flush=True)
    _check_sparse_rows(lib, 32, 4096, 64, torch.bfloat16, 2, seed=103, scale=1.0, chunk=chunk)


@pytest.mark.parametrize("p", [1, 2])
def test_config3_all_slices(lib, p):
    # causal long context, B*H = 16, N = 65536, D = 64, bf16, inputs scaled by 0.5
    print(f"case full config3 p={p}", flush=True)
    # the library's segments at this length: 128 tokens (order 1), 1024 tokens (order 2); a row with an
    # upstream gradient in every 128 (256) tokens covers every segment (512 / 256 + rows per slice)
    _check_sparse_rows(lib, 16, 65536, 64, torch.bfloat16, p, seed=110 + p, scale=0.5, seg=128 if p == 1 else 256)
    _check_running_mean(lib, 16, 65536, 64, torch.bfloat16, p, seed=120 + p)


@pytest.mark.parametrize("bh,n", [(40, 5000), (7, 9000), (96, 2304)])
def test_order1_runs_of_segments(lib, bh, n):
    """Order 1 on bf16 beyond 1024 tokens sums its 128-token segments in runs whose length follows the number of
    segments and batch*heads (3, 2 and 3 segments per run here; ragged last segment, last run of one or two
    segments, a whole number of runs): every segment holds a row with upstream gradient, so the part of every
    segment's state that comes from inside its run and the part that comes from the runs before / after it both
    enter o, dq, dk and dv."""
    print(f"case order-1 runs bh={bh} n={n}", flush=True)
    _check_sparse_rows(lib, bh, n, 64, torch.bfloat16, 1, seed=90 + bh, scale=0.7, seg=128)


def test_order1_runs_of_segments_dense_gradient(lib):
    """The same path with an upstream gradient on every row (runs of three segments), every result against the
    fp64 closed form."""
    from tests.parity import check_forward_backward
    print("case order-1 runs, dense dO", flush=True)
    check_forward_backward(lib, 40, 5000, 64, torch.bfloat16, DEV, mask=True, p=1, seed=77, scale=0.7, saved=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_config2_all_slices_sharp_temperature(lib, dtype):
    # temperature = sqrt(D) (what the reference's own tests use, test/test_einops_fastmax.py:77-225): scores of
    # order one, so the quadratic term carries real weight
    print(f"case full config2 tau=sqrt(D) dtype={dtype}", flush=True)
    _check_sparse_rows(lib, 32, 4096, 64, dtype, 2, seed=140, scale=1.0, tau_mult=1.0)
    _check_sparse_rows(lib, 32, 4096, 64, dtype, 2, seed=141, scale=1.0, tau_mult=1.0, chunk=1024)


@pytest.mark.parametrize("p", [1, 2])
def test_config3_all_slices_sharp_temperature(lib, p):
    print(f"case full config3 tau=sqrt(D) p={p}", flush=True)
    _check_sparse_rows(lib, 16, 65536, 64, torch.bfloat16, p, seed=150 + p, scale=0.5, seg=128 if p == 1 else 256, tau_mult=1.0)


@pytest.mark.parametrize("p", [1, 2])
def test_config3_prefix_is_independent_of_later_tokens(lib, p):
    print(f"case config3 prefix p={p}", flush=True)
    n, cut = 65536, 8192
    seg = 256 if p == 1 else 1024
    o, g, o2, g2 = _prefix_runs(lib, 16, n, cut, 64, torch.bfloat16, p, seed=130 + p, scale=0.5, chunk=seg)
    assert torch.equal(o[:, :cut], o2) and torch.equal(g[:, :cut], g2)
