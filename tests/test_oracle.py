"""Pins the CPU oracle (oracle/fastmax_oracle.py) without importing the reference.

The reference's own tests assert exactly two things for this path
(test/test_einops_fastmax.py): the factorised forward equals the quadratic
closed form to 1e-7 in float64 (:77-129) and the hand-written backward passes
gradcheck against it (:131-225); plus causality of the attention matrix
(:257-274).  Here the same statements are made for the oracle's restatements,
seeded, and the closed form itself is pinned by pure-Python loops and by
invariants that a dropped term, a wrong sign or a transposed operand breaks.
"""
import math

import pytest
import torch

from oracle import fastmax_oracle as O

torch.manual_seed(0)


def rnd(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=dtype)


def brute_force(q, k, v, mask, tau, c0, c1, c2):
    """Pure-Python triple loop for one head: the definition, nothing else."""
    nq, nk, d, dv = q.shape[0], k.shape[0], q.shape[1], v.shape[1]
    o = [[0.0] * dv for _ in range(nq)]
    g = [0.0] * nq
    for i in range(nq):
        last = nk - nq + i if mask else nk - 1
        for j in range(last + 1):
            s = sum(float(q[i, m]) * float(k[j, m]) for m in range(d)) / tau
            f = c0 + c1 * s + c2 * s * s
            g[i] += f
            for c in range(dv):
                o[i][c] += f * float(v[j, c])
        for c in range(dv):
            o[i][c] /= g[i]
    return torch.tensor(o, dtype=torch.float64), torch.tensor(g, dtype=torch.float64)


@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
def test_closed_form_vs_python_loops(mask, p):
    q, k, v = rnd(7, 3, seed=1), rnd(7, 3, seed=2), rnd(7, 4, seed=3)
    o, g = O.closed_form_forward(q, k, v, mask=mask, tau=1.7, p=p, a0=0.9, a1=1.1, a2=0.4)
    ob, gb = brute_force(q, k, v, mask, 1.7, 0.9, 1.1, 0.4 if p == 2 else 0.0)
    assert (o - ob).abs().max() < 1e-12
    assert (g - gb).abs().max() < 1e-12


def test_closed_form_tail_aligned_mask():
    # nk > nq: query i sees keys 0..nk-nq+i (fastmax_cuda_forward.cu:160-172)
    q, k, v = rnd(3, 2, seed=1), rnd(6, 2, seed=2), rnd(6, 2, seed=3)
    o, g = O.closed_form_forward(q, k, v, mask=True, tau=1.0, p=2)
    ob, gb = brute_force(q, k, v, True, 1.0, 1.0, 1.0, 0.5)
    assert (o - ob).abs().max() < 1e-12 and (g - gb).abs().max() < 1e-12


@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("norm_term", [1.0, 42.0])
def test_factorised_forward_equals_closed_form(mask, p, norm_term):
    # reference: test_einops_fastmax.py:77-129 (B=5,H=4,N=3,D=2, eps 1e-7); a longer
    # sequence and D != Dv-symmetric values are added so index mix-ups show.
    for (b, h, n, d) in [(5, 4, 3, 2), (2, 3, 17, 5)]:
        q, k, v = rnd(b, h, n, d, seed=4), rnd(b, h, n, d, seed=5), rnd(b, h, n, d, seed=6)
        tau = O.tau_einops(norm_term, d)
        o_ref, g_ref = O.closed_form_forward(q, k, v, mask=mask, tau=tau, p=p)
        o, g = O.factorised_forward(q, k, v, mask=mask, tau=tau, p=p)
        assert (o - o_ref).abs().max() < 1e-9
        assert (g - g_ref).abs().max() < 1e-9


@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("norm_term", [1.0, 42.0])
def test_factorised_backward_equals_autograd(mask, p, norm_term):
    # reference: gradcheck of the hand-written backward, test_einops_fastmax.py:131-225
    b, h, n, d = 2, 3, 9, 4
    q, k, v, go = (rnd(b, h, n, d, seed=s) for s in (7, 8, 9, 10))
    tau = O.tau_einops(norm_term, d)
    o, g, dq, dk, dv = O.closed_form_forward_backward(q, k, v, go, mask=mask, tau=tau, p=p)
    fq, fk, fv = O.factorised_backward(q, k, v, o, g, go, mask=mask, tau=tau, p=p)
    for a, b_ in ((fq, dq), (fk, dk), (fv, dv)):
        assert O.rel_l2(a, b_) < 1e-10


@pytest.mark.parametrize("mask", [False, True])
def test_autograd_gradient_vs_finite_differences(mask):
    # independent of autograd: central differences of sum(o * dO)
    n, d = 5, 3
    q, k, v, go = (rnd(1, 1, n, d, seed=s) for s in (11, 12, 13, 14))
    _, _, dq, dk, dv = O.closed_form_forward_backward(q, k, v, go, mask=mask, tau=1.3, p=2,
                                                      a0=1.0, a1=0.8, a2=0.3)

    def loss(q_, k_, v_):
        o, _ = O.closed_form_forward(q_, k_, v_, mask=mask, tau=1.3, p=2, a0=1.0, a1=0.8, a2=0.3)
        return float((o * go).sum())

    eps = 1e-6
    for idx, (x, dx) in enumerate(((q, dq), (k, dk), (v, dv))):
        num = torch.zeros_like(x)
        for t in range(n):
            for c in range(d):
                xp = x.clone(); xp[0, 0, t, c] += eps
                xm = x.clone(); xm[0, 0, t, c] -= eps
                args_p = [q, k, v]; args_m = [q, k, v]
                args_p[idx] = xp; args_m[idx] = xm
                num[0, 0, t, c] = (loss(*args_p) - loss(*args_m)) / (2 * eps)
        assert (num - dx).abs().max() < 1e-7


@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
def test_manual_blocked_backward_equals_autograd(mask, p):
    b, h, n, d = 1, 2, 37, 4
    q, k, v, go = (rnd(b, h, n, d, seed=s) for s in (15, 16, 17, 18))
    ref = O.closed_form_forward_backward(q, k, v, go, mask=mask, tau=2.0, p=p, a0=1.0, a1=0.7, a2=0.6)
    got = O.manual_backward_blocked(q, k, v, go, mask=mask, tau=2.0, p=p, a0=1.0, a1=0.7, a2=0.6,
                                    block=8)
    for a, b_ in zip(got, ref):
        assert O.rel_l2(a, b_) < 1e-12


@pytest.mark.parametrize("p", [1, 2])
def test_sampled_rows_equal_autograd_with_sparse_upstream_gradient(p):
    # dO zero outside a few query rows: autograd through the full closed form must give the
    # same o, g and dq at those rows, zero dq elsewhere, and the same full dk, dv
    bh, n, d = 3, 41, 5
    q, k, v, go = (rnd(1, bh, n, d, seed=s)[0] for s in (31, 32, 33, 34))
    rows = torch.tensor([0, 7, 8, 23, 40])
    sparse = torch.zeros_like(go)
    sparse[:, rows] = go[:, rows]
    o, g, dq, dk, dv = O.closed_form_forward_backward(q, k, v, sparse, mask=True, tau=1.7, p=p, a0=0.9, a1=0.7, a2=0.6)
    got = O.sampled_rows_forward_backward(q, k, v, rows, go[:, rows], tau=1.7, p=p, a0=0.9, a1=0.7, a2=0.6)
    other = torch.ones(n, dtype=torch.bool); other[rows] = False
    assert dq[:, other].abs().max() == 0
    for a, b_ in zip(got, (o[:, rows], g[:, rows], dq[:, rows], dk, dv)):
        assert O.rel_l2(a, b_) < 1e-12


def test_causality_and_first_token():
    # reference: test_fastmax_iscausal (:257-274): a[i, j] == 0 for j > i
    q, k, v = rnd(1, 2, 6, 3, seed=19), rnd(1, 2, 6, 3, seed=20), rnd(1, 2, 6, 3, seed=21)
    o, g, a = O.closed_form_forward(q, k, v, mask=True, tau=O.tau_einops(42, 3), p=2, return_attn=True)
    assert torch.all(a.triu(1) == 0)
    assert torch.allclose(a.sum(-1), torch.ones_like(g))
    assert torch.allclose(o[..., 0, :], v[..., 0, :])         # first token only sees itself
    # future keys/values do not influence earlier outputs (factorised path too)
    k2, v2 = k.clone(), v.clone()
    k2[..., 4:, :] += 3.0; v2[..., 4:, :] -= 5.0
    o2, _ = O.factorised_forward(q, k2, v2, mask=True, tau=O.tau_einops(42, 3), p=2)
    assert torch.allclose(o2[..., :4, :], o[..., :4, :], atol=1e-12)


def test_invariants():
    q, k, v = rnd(1, 1, 8, 4, seed=22), rnd(1, 1, 8, 4, seed=23), rnd(1, 1, 8, 4, seed=24)
    tau = 2.0
    # rows of the attention matrix sum to one: constant values stay constant
    o, _ = O.closed_form_forward(q, k, torch.full_like(v, 3.25), mask=True, tau=tau, p=2)
    assert torch.allclose(o, torch.full_like(o, 3.25))
    # a1 = a2 = 0: causal output is the running mean of v
    o, g = O.closed_form_forward(q, k, v, mask=True, tau=tau, p=2, a0=1.0, a1=0.0, a2=0.0)
    assert torch.allclose(o, torch.cumsum(v, 2) / torch.arange(1, 9).view(1, 1, 8, 1))
    assert torch.allclose(g, torch.arange(1, 9, dtype=torch.float64).view(1, 1, 8))
    # unmasked output is invariant to a permutation of the (key, value) pairs
    perm = torch.randperm(8, generator=torch.Generator().manual_seed(1))
    o1, _ = O.factorised_forward(q, k, v, mask=False, tau=tau, p=2)
    o2, _ = O.factorised_forward(q, k[:, :, perm], v[:, :, perm], mask=False, tau=tau, p=2)
    assert torch.allclose(o1, o2, atol=1e-12)
    # order 2 with Taylor coefficients: g > 0 because f(s) = ((s+1)^2 + 1)/2
    _, g = O.closed_form_forward(5 * q, 5 * k, v, mask=True, tau=1.0, p=2)
    assert torch.all(g > 0)
    # output is linear in v
    oa, _ = O.closed_form_forward(q, k, v, mask=True, tau=tau, p=2)
    ob, _ = O.closed_form_forward(q, k, 2 * v + 1, mask=True, tau=tau, p=2)
    assert torch.allclose(ob, 2 * oa + 1)


def test_dv_is_reversed_forward():
    # dV_j = sum_i M_ij f(s_ij) ghat_i: the un-normalised forward run right-to-left
    # with (q <-> k, v -> ghat)
    n, d = 9, 3
    q, k, v, go = (rnd(1, 1, n, d, seed=s) for s in (25, 26, 27, 28))
    o, g, _, _, dv = O.closed_form_forward_backward(q, k, v, go, mask=True, tau=1.5, p=2)
    gh = go / g.unsqueeze(-1)
    flip = lambda t: torch.flip(t, (2,))
    of, gf = O.closed_form_forward(flip(k), flip(q), flip(gh), mask=True, tau=1.5, p=2)
    assert torch.allclose(flip(of * gf.unsqueeze(-1)), dv, atol=1e-12)


def test_extension_semantics_match_einops_front():
    # einops(normalize_term=c) == extension(temperature=c*sqrt(D), a=(1,1,1/2))
    # (fastattention_einops.py:79-82 + fastmax_cuda_forward.cu:288)
    b, h, n, d = 2, 2, 6, 4
    q, k, v = rnd(b, h, n, d, seed=29), rnd(b, h, n, d, seed=30), rnd(b, h, n, d, seed=31)
    o_e, g_e = O.factorised_forward(q, k, v, mask=True, tau=O.tau_einops(8, d), p=2)
    to_ext = lambda t: t.reshape(b * h, n, d).permute(1, 0, 2).contiguous()
    out = O.extension_forward(to_ext(q), to_ext(k), to_ext(v), mask=True,
                              temperature=8 * math.sqrt(d), a0=1.0, a1=1.0, a2=0.5, p=2)
    assert out.shape == (n, b * h, d + 1)
    assert torch.allclose(out[..., :d], to_ext(o_e), atol=1e-12)
    assert torch.allclose(out[..., d], g_e.reshape(b * h, n).t(), atol=1e-12)
    # backward of the extension: gradients w.r.t. q and the already-scaled k
    go = rnd(n, b * h, d, seed=32)
    t = 8 * math.sqrt(d)
    gq, gk, gv = O.extension_backward(to_ext(q), to_ext(k) / t, to_ext(v), go, mask=True,
                                      a0=1.0, a1=1.0, a2=0.5, p=2)
    from_ext = lambda x: x.permute(1, 0, 2).reshape(b, h, n, d)
    _, _, dq, dk, dv = O.closed_form_forward_backward(q, k, v, from_ext(go), mask=True,
                                                      tau=t, p=2)
    assert O.rel_l2(from_ext(gq), dq) < 1e-12
    assert O.rel_l2(from_ext(gk) / t, dk) < 1e-12        # the wrapper's gradk / t (model.py:74)
    assert O.rel_l2(from_ext(gv), dv) < 1e-12


def test_normalisers():
    x, y = rnd(2, 3, 7, 5, seed=33), rnd(2, 3, 7, 5, seed=34)
    a, b = O.normalize_feature_mean(x, y)
    f64 = dict(dtype=torch.float64)
    assert torch.allclose(a.sum(-1), torch.zeros(2, 3, 7, **f64), atol=1e-12)
    assert torch.allclose(a.norm(dim=-1).amax(-1), torch.ones(2, 3, **f64))
    a, b = O.normalize_token_mean(x, y)
    assert torch.allclose(b.sum(-2), torch.zeros(2, 3, 5, **f64), atol=1e-12)
    assert torch.allclose(b.norm(dim=-1).amax(-1), torch.ones(2, 3, **f64))
    c = O.normalize_lim(x, lim=2.0)
    assert torch.allclose(c.norm(dim=-1).amax(-1), torch.full((2, 3), 2.0, **f64))
    # a pure per-(b,h) rescale: undoing it gives x back
    assert torch.allclose(c[0, 0] * x[0, 0].norm(dim=-1).max() / 2.0, x[0, 0])


def test_score_function_front():
    q, k, v = rnd(1, 2, 6, 4, seed=35), rnd(1, 2, 6, 4, seed=36), rnd(1, 2, 6, 4, seed=37)
    o = O.score_function_fastmax(q, k, v, mask=True, denum_term=8, normalize=0, p=2)
    o_ref, _ = O.factorised_forward(q, k, v, mask=True, tau=8 * 2.0, p=2)
    assert torch.allclose(o, o_ref, atol=1e-12)
    o = O.score_function_fastmax(q, k, v, mask=None, denum_term=8, normalize=1, p=1)
    qn, kn = O.normalize_token_mean(q, k)
    o_ref, _ = O.factorised_forward(qn, kn, v, mask=False, tau=1.0, p=1)
    assert torch.allclose(o, o_ref, atol=1e-12)
    o, a = O.score_function_fastmax(q, k, v, mask=None, create_attn_matrix=True)
    assert torch.allclose(a.sum(-1), torch.ones(1, 2, 6, dtype=torch.float64))
    assert torch.allclose(a @ v, o)


def test_attn_matrix_tensor_mask():
    """The debug branch takes the mask as a tensor (reference score_function.py:243-244): a lower-triangular
    one reproduces the causal closed form, an arbitrary one is checked entry by entry with plain loops."""
    q, k, v = rnd(1, 2, 6, 4, seed=41), rnd(1, 2, 6, 4, seed=42), rnd(1, 2, 6, 4, seed=43)
    tril = torch.ones(6, 6).tril()
    o, a = O.score_function_fastmax(q, k, v, mask=tril, create_attn_matrix=True)
    o_ref, _ = O.closed_form_forward(q, k, v, mask=True, tau=8 * 2.0, p=2)
    assert torch.allclose(o, o_ref, atol=1e-12)
    g = torch.Generator().manual_seed(5)
    m = (torch.rand(6, 6, generator=g) < 0.6).float()
    m[:, 0] = 1                                            # no empty row
    o, a = O.score_function_fastmax(q, k, v, mask=m, create_attn_matrix=True)
    for h in range(2):
        for i in range(6):
            w = []
            for j in range(6):
                s = sum(float(q[0, h, i, c]) * float(k[0, h, j, c]) for c in range(4)) / 16.0
                w.append((1 + s + 0.5 * s * s) if m[i, j] != 0 else 0.0)
            tot = sum(w)
            for j in range(6):
                assert abs(float(a[0, h, i, j]) - w[j] / tot) < 1e-12
            for c in range(4):
                want = sum(w[j] * float(v[0, h, j, c]) for j in range(6)) / tot
                assert abs(float(o[0, h, i, c]) - want) < 1e-12


def test_dormant_steps_known_answers():
    """The two steps the reference ships switched off (fastmax_cuda_forward.cu:289, :340-349, :443), worked by hand:
    for nk = 3 the table rows met by tokens 0, 1, 2 are (l + 3) % 5 = 3, 4, 0."""
    k = torch.tensor([[[2.0, 4.0], [6.0, 8.0], [10.0, 12.0]]])
    rpe = torch.tensor([[0.5, 0.25], [100.0, 100.0], [100.0, 100.0], [1.0, 2.0], [3.0, 4.0]])
    got = O.apply_rpe_and_temp(k, rpe, temperature=2.0)
    want = torch.tensor([[[1.0 + 1.0, 2.0 + 2.0], [3.0 + 3.0, 4.0 + 4.0], [5.0 + 0.5, 6.0 + 0.25]]], dtype=torch.float64)
    assert torch.equal(got, want)
    assert torch.equal(O.apply_rpe_and_temp(k, rpe, temperature=2.0, add_rpe=False), k.double() / 2.0)
    # every table row but one is met at most once, and rows nk .. 2nk-2 come first
    n = 7
    idx = [(l + n) % (2 * n - 1) for l in range(n)]
    assert idx == list(range(n, 2 * n - 1)) + [0]
    o = torch.tensor([[1.0, -2.0], [4.0, 0.5]])
    noise = torch.tensor([[0.5, 1.0], [-1.0, 2.0]])
    assert torch.equal(O.apply_dropout(o, noise, 0.0), o.double())
    assert torch.equal(O.apply_dropout(o, noise, 0.5), torch.tensor([[1.25, -3.0], [2.0, 1.0]], dtype=torch.float64))
