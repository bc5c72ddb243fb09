"""GPU tests of the torch binding (`fastmax_cuda`) and the operator fronts, against the oracle."""
import math

import pytest
import torch

from oracle import fastmax_oracle as O
from tests.parity import TOL, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ext():
    from reproducing_fastmax_results_amd import fastmax_cuda
    return fastmax_cuda


@pytest.fixture(scope="module")
def sf():
    from reproducing_fastmax_results_amd.attention_mechanisms import score_function
    return score_function


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
def test_legacy_forwardpass_backwardpass(ext, mask, p):
    """Reference call sequence of transformer/model.py:29-74 on (n, b*h, d) fp32 tensors."""
    n, bh, d, t = 300, 6, 32, 3.7
    q, k, v, go = (rnd(n, bh, d, seed=s) for s in (1, 2, 3, 4))
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    noise = torch.zeros_like(qd)
    rpe = torch.zeros(2 * n - 1, d, device=DEV)
    out = ext.forwardpass(qd, kd, vd, noise, rpe, mask, 0.1, False, t, 1.0, 1.0, 0.5, 1.0, p)
    assert out.shape == (n, bh, d + 1) and out.dtype == torch.float32
    # like the reference, k is left divided by the temperature (fastmax_cuda_forward.cu:288)
    assert torch.allclose(kd.cpu(), k / t, rtol=1e-6, atol=1e-7)
    assert torch.equal(qd.cpu(), q)
    ref = O.extension_forward(q, k, v, mask=mask, temperature=t, a0=1.0, a1=1.0, a2=0.5, p=p)
    assert rel_err(out, ref) < 1e-5
    gq, gk, gv = ext.backwardpass(qd, kd, vd, out, go.to(DEV), mask, 1.0, 1.0, 0.5, p)
    rq, rk, rv = O.extension_backward(q, k / t, v, go, mask=mask, a0=1.0, a1=1.0, a2=0.5, p=p)
    for a, b in ((gq, rq), (gk, rk), (gv, rv)):
        assert rel_err(a, b) < 1e-5


def test_legacy_normalize_flag(ext):
    n, bh, d = 130, 4, 64
    q, k, v = (rnd(n, bh, d, seed=s) for s in (5, 6, 7))
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out = ext.forwardpass(qd, kd, vd, torch.zeros_like(qd), torch.zeros(2 * n - 1, d, device=DEV), True, 0.0, True,
                          2.0, 1.0, 1.0, 0.5, 1.5, 2)
    qn = O.normalize_lim(q.permute(1, 0, 2).double(), 1.5).permute(1, 0, 2)
    kn = O.normalize_lim(k.permute(1, 0, 2).double(), 1.5).permute(1, 0, 2)
    assert rel_err(qd, qn) < 1e-5 and rel_err(kd, kn) < 1e-5
    ref = O.extension_forward(qn, kn, v, mask=True, temperature=1.0, a0=1.0, a1=1.0, a2=0.5, p=2)
    assert rel_err(out, ref) < 1e-5


def test_legacy_errors(ext):
    n, bh, d = 64, 2, 32
    q = torch.randn(n, bh, d, device=DEV)
    z = torch.zeros_like(q)
    rpe = torch.zeros(2 * n - 1, d, device=DEV)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.forwardpass(q.permute(1, 0, 2), q, q, z, rpe, True, 0.0, False, 1.0, 1.0, 1.0, 0.5, 1.0, 2)
    with pytest.raises(RuntimeError, match="CUDA"):
        ext.forwardpass(q.cpu(), q, q, z, rpe, True, 0.0, False, 1.0, 1.0, 1.0, 0.5, 1.0, 2)
    with pytest.raises(RuntimeError, match="unsupported"):
        ext.forwardpass(q, q, q, z, rpe, True, 0.0, False, 1.0, 1.0, 1.0, 0.5, 1.0, 3)
    q48 = torch.randn(n, bh, 48, device=DEV)
    with pytest.raises(RuntimeError, match="unsupported"):
        ext.forwardpass(q48, q48, q48, torch.zeros_like(q48), rpe, True, 0.0, False, 1.0, 1.0, 1.0, 0.5, 1.0, 2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("four_d", [False, True])
def test_autograd_wrapper(sf, dtype, four_d):
    b, h, n, d, t = 2, 3, 700, 64, 11.0
    shape = (b, h, n, d) if four_d else (b * h, n, d)
    q, k, v, go = (rnd(*shape, seed=s).to(dtype) for s in (8, 9, 10, 11))
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    noise = torch.zeros_like(qd)
    rpe = sf.rpe_matrix_creator(n, d, DEV, torch.float32)
    o = sf.FASTMultiHeadAttention_Function.apply(qd, kd, vd, noise, rpe, True, 0.1, False, t, 1.0, 1.0, 0.5, 1.0, 2)
    assert o.shape == shape
    o.backward(go.to(DEV))
    ref = O.manual_backward_blocked(q.double(), k.double(), v.double(), go.double(), mask=True, tau=t, p=2)
    assert rel_err(o, ref[0]) < TOL[dtype]
    for got, want in ((qd.grad, ref[2]), (kd.grad, ref[3]), (vd.grad, ref[4])):
        assert rel_err(got, want) < TOL[dtype]
    # module form and the reference's model-side call (transformer/model.py:301-303)
    o2 = sf.fastmax_custom(qd, kd, vd, noise, rpe, True, 0.1, False, t, 1.0, 1.0, 0.5, 1.0, 2)
    assert torch.equal(o2, o)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_normalised_attention_function(sf, dtype):
    """FastmaxNormAttention: normalisation folded into the kernels, gradients with respect to the raw q and k
    (fp64 autograd through lim * x / max-norm and the closed form); and the reference-style wrapper with
    normalize=True, whose gradients are those with respect to the normalised tensors."""
    b, h, n, d, lim = 2, 3, 600, 64, 1.3
    q, k, v, go = (rnd(b, n, h * d, seed=s).to(dtype).to(DEV).view(b, n, h, d).transpose(1, 2) for s in (44, 45, 46, 47))
    qd, kd, vd = (x.detach().clone().requires_grad_(True) for x in (q, k, v))
    o = sf.FastmaxNormAttention.apply(qd, kd, vd, True, lim, 1.0, 1.0, 1.0, 0.5, 2)
    o.backward(go)
    q64, k64, v64 = (x.double().cpu().contiguous().requires_grad_(True) for x in (q, k, v))
    oo, _ = O.closed_form_forward(O.normalize_lim(q64, lim), O.normalize_lim(k64, lim), v64, mask=True, tau=1.0, p=2)
    rq, rk, rv = torch.autograd.grad(oo, (q64, k64, v64), go.double().cpu())
    assert rel_err(o, oo) < TOL[dtype]
    for got, want in ((qd.grad, rq), (kd.grad, rk), (vd.grad, rv)):
        assert rel_err(got, want) < TOL[dtype]
    # the reference's call: normalize inside, gradients with respect to the normalised q and k
    qe, ke, ve = (x.detach().clone().requires_grad_(True) for x in (q, k, v))
    o2 = sf.FASTMultiHeadAttention_Function.apply(qe, ke, ve, None, None, True, 0.0, True, 1.0, 1.0, 1.0, 0.5, lim, 2)
    o2.backward(go)
    assert torch.equal(o2, o)
    qn, kn = O.normalize_lim(q.double().cpu(), lim), O.normalize_lim(k.double().cpu(), lim)
    ref = O.manual_backward_blocked(qn.contiguous(), kn.contiguous(), v.double().cpu().contiguous(), go.double().cpu().contiguous(),
                                    mask=True, tau=1.0, p=2)
    for got, want in ((qe.grad, ref[2]), (ke.grad, ref[3]), (ve.grad, ref[4])):
        assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_head_per_batch_projection_layout(sf, ext, dtype):
    """(b, n, 1*d) projections viewed as (b, 1, n, d): stride(1) of that view is d, not the distance between
    the batches; the binding must address batch i at i * n * d (heads_per_block = 1 in the model)."""
    b, n, d, t = 3, 200, 64, 9.0
    q, k, v, go = (rnd(b, n, d, seed=s).to(dtype).to(DEV).view(b, n, 1, d).transpose(1, 2) for s in (40, 41, 42, 43))
    assert q.shape == (b, 1, n, d) and q.stride(1) == d
    qd, kd, vd = (x.detach().clone().requires_grad_(True) for x in (q, k, v))   # clone keeps the strides
    assert qd.stride() == q.stride()
    noise, rpe = torch.zeros_like(qd), sf.rpe_matrix_creator(n, d, DEV, torch.float32)
    o = sf.FASTMultiHeadAttention_Function.apply(qd, kd, vd, noise, rpe, True, 0.0, False, t, 1.0, 1.0, 0.5, 1.0, 2)
    o.backward(go)
    ref = O.manual_backward_blocked(*(x.double().cpu().contiguous() for x in (q, k, v, go)), mask=True, tau=t, p=2)
    assert rel_err(o, ref[0]) < TOL[dtype]
    for got, want in ((qd.grad, ref[2]), (kd.grad, ref[3]), (vd.grad, ref[4])):
        assert rel_err(got, want) < TOL[dtype]
    o1, g1 = ext.forward_ex(q, k, v, True, 1.0 / t, 1.0, 1.0, 0.5, 2, 0, 0)
    o2, g2 = ext.forward_ex(q.contiguous(), k.contiguous(), v.contiguous(), True, 1.0 / t, 1.0, 1.0, 0.5, 2, 0, 0)
    assert torch.equal(o1, o2) and torch.equal(g1, g2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_transposed_projection_layout(sf, ext, dtype):
    """(b, n, h*d) projections viewed as (b, h, n, d) - the layout Attention.forward produces
    (transformer/model.py:283-285) - are consumed through batch and head strides, without a copy,
    the result comes back in the same memory order (its transpose to (b, n, h*d) is a view), and
    so do the gradients."""
    b, h, n, d = 2, 4, 260, 32
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    q, k, v, go = (rnd(b, n, h * d, seed=s).to(dtype).to(DEV).view(b, n, h, d).transpose(1, 2) for s in (12, 13, 14, 15))
    assert not q.is_contiguous()
    o = sf.fastmax_einops(q, k, v, mask=True, normalize_term=8, p=2)
    qd, kd, vd, god = (x.double().cpu() for x in (q, k, v, go))
    ref = O.closed_form_forward_backward(qd, kd, vd, god, mask=True, tau=O.tau_einops(8, d), p=2)
    assert rel_err(o, ref[0]) < tol
    assert o.transpose(1, 2).is_contiguous()          # (b, n, h, d) in memory
    # the strided entry points directly: same numbers as on contiguous copies, bit for bit
    inv_tau = 1.0 / O.tau_einops(8, d)
    o1, g1, ws = ext.forward_save(q, k, v, True, inv_tau, 1.0, 1.0, 0.5, 2, 0, 0)
    o2, g2 = ext.forward_ex(q.contiguous(), k.contiguous(), v.contiguous(), True, inv_tau, 1.0, 1.0, 0.5, 2, 0, 0)
    assert torch.equal(o1, o2) and torch.equal(g1, g2)
    dq, dk, dv = ext.backward_saved(q, k, v, o1, g1, go, ws, True, inv_tau, 1.0, 1.0, 0.5, 2, 0, 0)
    # (the backward on a kept forward workspace also reads what bf16 rounding took from o there, so its twin on
    # contiguous copies is the same pair of calls, not backward_ex)
    o3, g3, ws3 = ext.forward_save(q.contiguous(), k.contiguous(), v.contiguous(), True, inv_tau, 1.0, 1.0, 0.5, 2, 0, 0)
    eq, ek, ev = ext.backward_saved(q.contiguous(), k.contiguous(), v.contiguous(), o3, g3, go.contiguous(), ws3, True,
                                    inv_tau, 1.0, 1.0, 0.5, 2, 0, 0)
    assert torch.equal(dq, eq) and torch.equal(dk, ek) and torch.equal(dv, ev)
    assert dq.transpose(1, 2).is_contiguous() and dk.transpose(1, 2).is_contiguous()
    for got, want in zip((dq, dk, dv), ref[2:]):
        assert rel_err(got, want) < tol


@pytest.mark.parametrize("normalize", [0, 1])
@pytest.mark.parametrize("mask", [None, True])
@pytest.mark.parametrize("p", [1, 2])
def test_score_function_front(sf, normalize, mask, p):
    """fastmax(q,k,v,mask,denum_term,normalize,p) including gradients through the
    token-mean / max-norm normalisation (score_function.py:40-57)."""
    b, h, n, d = 1, 2, 150, 32
    q, k, v, go = (rnd(b, h, n, d, seed=s) for s in (15, 16, 17, 18))
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    o = sf.fastmax(qd, kd, vd, mask=mask, denum_term=8, normalize=normalize, p=p)
    o.backward(go.to(DEV))
    qr, kr, vr = (x.double().requires_grad_(True) for x in (q, k, v))
    oref = O.score_function_fastmax(qr, kr, vr, mask=mask, denum_term=8, normalize=normalize, p=p)
    oref.backward(go.double())
    assert rel_err(o, oref) < 1e-5
    for got, want in ((qd.grad, qr.grad), (kd.grad, kr.grad), (vd.grad, vr.grad)):
        assert rel_err(got, want) < 2e-5      # the fp32 normalisation backward pass on top of the kernels


def test_rpe_matrix_structured(sf):
    """Sinusoidal relative-position table (reference transformer/model.py:230-241): row n - 1 + t holds
    position -t, row n - 1 - t position +t; checked against the closed form entry by entry."""
    n, d = 9, 32
    rpe = sf.rpe_matrix_creator(n, d, DEV, torch.float32, structured=True).cpu()
    assert rpe.shape == (2 * n - 1, d)
    for row in range(2 * n - 1):
        pos = float(n - 1 - row)
        for c in range(0, d, 2):
            w = math.exp(-c * math.log(10000.0) / d)
            assert abs(float(rpe[row, c]) - math.sin(pos * w)) < 1e-5
            assert abs(float(rpe[row, c + 1]) - math.cos(pos * w)) < 1e-5
    rnd_rpe = sf.rpe_matrix_creator(n, d, DEV, torch.float32, structured=False, is_zero=False)
    assert rnd_rpe.shape == (2 * n - 1, d) and float(rnd_rpe.abs().sum()) > 0


def test_create_attn_matrix_debug_path(sf):
    q, k, v = (rnd(1, 2, 40, 32, seed=s).to(DEV) for s in (19, 20, 21))
    o, a = sf.fastmax(q, k, v, mask=True, p=2, create_attn_matrix=True)
    assert torch.all(a.triu(1) == 0)                      # reference test_fastmax_iscausal
    assert torch.allclose(a.sum(-1), torch.ones_like(a.sum(-1)), atol=1e-5)
    o2 = sf.fastmax(q, k, v, mask=True, denum_term=8, p=2)
    assert rel_err(o, o2) < 1e-5
    # the reference passes the mask of this branch as a tensor (score_function.py:243-244)
    tril = torch.ones(40, 40, device=DEV).tril()
    o3, a3 = sf.fastmax(q, k, v, mask=tril, p=2, create_attn_matrix=True)
    assert torch.equal(a3, a)
    m = (torch.rand(40, 40, generator=torch.Generator().manual_seed(3)) < 0.5).float()
    m[:, 0] = 1
    o4, a4 = sf.fastmax(q, k, v, mask=m.to(DEV), p=2, create_attn_matrix=True)
    ow, aw = O.score_function_fastmax(q.double().cpu(), k.double().cpu(), v.double().cpu(), mask=m.double(),
                                      create_attn_matrix=True)
    assert rel_err(a4, aw) < 1e-5 and rel_err(o4, ow) < 1e-5


@pytest.mark.parametrize("centre", [0, 1, 2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_normalize_kernel(ext, centre, dtype):
    x = rnd(3, 2, 333, 64, seed=22).to(dtype)
    y = ext.normalize(x.to(DEV), centre, True, 2.0)
    xd = x.double()
    if centre == 1:
        ref = O.normalize_feature_mean(xd, xd)[0] * 2.0
    elif centre == 2:
        ref = O.normalize_token_mean(xd, xd)[0] * 2.0
    else:
        ref = O.normalize_lim(xd, 2.0)
    assert rel_err(y, ref) < (1e-5 if dtype == torch.float32 else 1e-2)


def _normalize_ref(xd, centre, scale):
    if centre == 1:
        return O.normalize_feature_mean(xd, xd)[0] * scale
    if centre == 2:
        return O.normalize_token_mean(xd, xd)[0] * scale
    return O.normalize_lim(xd, scale)


@pytest.mark.parametrize("centre", [0, 1, 2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(3, 2, 333, 64), (5, 700, 32)])
def test_normalize_backward_kernel(ext, centre, dtype, shape):
    """Gradient of the normalisation pass against autograd (fp64) through the oracle's formula."""
    print(f"case normalize backward centre={centre} dtype={dtype} shape={shape}", flush=True)
    x = rnd(*shape, seed=40).to(dtype)
    dy = rnd(*shape, seed=41).to(dtype)
    dx = ext.normalize_backward(x.to(DEV), dy.to(DEV), centre, True, 2.0)
    xd = x.double().requires_grad_(True)
    _normalize_ref(xd, centre, 2.0).backward(dy.double())
    assert dx.shape == x.shape
    assert rel_err(dx, xd.grad) < (1e-5 if dtype == torch.float32 else 1e-2)
    # without the max-norm division the pass is linear: dx = scale * centred dy
    dx0 = ext.normalize_backward(x.to(DEV), dy.to(DEV), centre, False, 0.5)
    dyd = dy.double()
    want = 0.5 * (dyd - (dyd.mean(-1, keepdim=True) if centre == 1 else dyd.mean(-2, keepdim=True) if centre == 2 else 0))
    assert rel_err(dx0, want) < (1e-5 if dtype == torch.float32 else 1e-2)


def test_normalize_backward_equal_norms_and_repeat(ext):
    """Two tokens share the largest norm, in different workgroups: the gradient's one-token term goes
    to the first of them (the rule the header states), and two runs give the same bits."""
    n, d = 1000, 64
    x, dy = rnd(2, n, d, seed=44), rnd(2, n, d, seed=45)
    x[:, 700] = 50.0 * x[:, 700] / x[:, 700].norm(dim=-1, keepdim=True)
    x[:, 130] = x[:, 700]
    dx = ext.normalize_backward(x.to(DEV), dy.to(DEV), 0, True, 1.0)
    again = ext.normalize_backward(x.to(DEV), dy.to(DEV), 0, True, 1.0)
    assert torch.equal(dx, again)
    xd, dyd = x.double(), dy.double()
    m = xd.norm(dim=-1).amax(-1)                                    # (bh,)
    plain = dyd / m[:, None, None]                                  # every token but the first largest one
    assert rel_err(dx[:, 700], plain[:, 700]) < 1e-5
    spike = (dx.cpu().double() - plain)[:, 130]
    want = -((dyd * xd).sum((-1, -2)) / m ** 3)[:, None] * xd[:, 130]
    assert rel_err(spike, want) < 1e-4


def test_normalize_backward_on_projection_layout(ext):
    """x and dy as the (b, h, n, d) views of (b, n, h*d) projections: no copies, dx in x's layout."""
    b, h, n, d = 2, 4, 130, 64
    xp, dyp = rnd(b, n, h * d, seed=42).to(DEV), rnd(b, n, h * d, seed=43).to(DEV)
    x, dy = (t.view(b, n, h, d).transpose(1, 2) for t in (xp, dyp))
    dx = ext.normalize_backward(x, dy, 2, True, 1.0)
    assert dx.transpose(1, 2).is_contiguous()
    xd = x.cpu().double().requires_grad_(True)
    _normalize_ref(xd, 2, 1.0).backward(dy.cpu().double())
    assert rel_err(dx, xd.grad) < 1e-5


@pytest.mark.parametrize("nq", [1, 200])
def test_autograd_wrapper_with_cached_keys(sf, nq):
    """Causal call with fewer queries than keys (the queries are the last tokens, the other keys a
    cache: fastmax_cuda_forward.cu:161-172), through the autograd wrapper, gradients included."""
    b, h, nk, d, t = 2, 2, 450, 64, 9.0
    q = rnd(b, h, nq, d, seed=60)
    k, v = rnd(b, h, nk, d, seed=61), rnd(b, h, nk, d, seed=62)
    go = rnd(b, h, nq, d, seed=63)
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    o = sf.FASTMultiHeadAttention_Function.apply(qd, kd, vd, None, None, True, 0.0, False, t, 1.0, 1.0, 0.5, 1.0, 2)
    o.backward(go.to(DEV))
    ref = O.closed_form_forward_backward(q, k, v, go, mask=True, tau=t, p=2)
    assert rel_err(o, ref[0]) < 1e-5
    for got, want in ((qd.grad, ref[2]), (kd.grad, ref[3]), (vd.grad, ref[4])):
        assert rel_err(got, want) < 1e-5
    # the last rows of the full square problem are the same thing
    qf = torch.cat([rnd(b, h, nk - nq, d, seed=64), q], dim=2).to(DEV)
    of = sf.FASTMultiHeadAttention_Function.apply(qf, kd.detach(), vd.detach(), None, None, True, 0.0, False, t,
                                                  1.0, 1.0, 0.5, 1.0, 2)
    assert rel_err(o, of[:, :, nk - nq:]) < 1e-5


@pytest.mark.parametrize("d", [20, 48])
@pytest.mark.parametrize("normalize", [False, True])
def test_other_head_sizes_run_padded(sf, d, normalize):
    """Head sizes between the two the kernels are built for: zero-padded inside the autograd
    function, results and gradients of the caller's shape, against the oracle at the true size."""
    b, h, n, t = 2, 3, 333, 5.0
    q, k, v, go = (rnd(b, h, n, d, seed=s) for s in (70, 71, 72, 73))
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    o = sf.FASTMultiHeadAttention_Function.apply(qd, kd, vd, None, None, True, 0.0, normalize, t, 1.0, 1.0, 0.5, 1.5, 2)
    assert o.shape == (b, h, n, d)
    o.backward(go.to(DEV))
    qr, kr, vr = (x.double().requires_grad_(True) for x in (q, k, v))
    qn, kn = (O.normalize_lim(qr, 1.5), O.normalize_lim(kr, 1.5)) if normalize else (qr, kr)
    qn.retain_grad(); kn.retain_grad()
    oref, _ = O.closed_form_forward(qn, kn, vr, mask=True, tau=t, p=2)
    oref.backward(go.double())
    assert rel_err(o, oref) < 1e-5
    # like the reference, the function returns the gradients with respect to the normalised q and k
    for got, want in ((qd.grad, qn.grad), (kd.grad, kn.grad), (vd.grad, vr.grad)):
        assert got.shape == want.shape and rel_err(got, want) < 1e-5
    # the differentiable normalisation on its own, token-mean centring
    x = rnd(b, h, n, d, seed=74)
    xd = x.to(DEV).requires_grad_(True)
    y = sf.FastmaxNormalize.apply(xd, sf.CENTRE_TOKEN, 2.0)
    y.backward(go.to(DEV))
    xr = x.double().requires_grad_(True)
    yr = O.normalize_token_mean(xr, xr)[0] * 2.0
    yr.backward(go.double())
    assert rel_err(y, yr) < 1e-5 and rel_err(xd.grad, xr.grad) < 1e-5
    with pytest.raises(RuntimeError, match="unsupported head size"):
        sf.FASTMultiHeadAttention_Function.apply(*(rnd(1, 1, 8, 80).to(DEV) for _ in range(3)))



@pytest.mark.parametrize("d", [100, 128])
@pytest.mark.parametrize("normalize", [False, True])
def test_wide_heads_on_bf16(sf, d, normalize):
    """Heads of up to 128 on bfloat16 tensors through the autograd wrapper (100: zero-padded to 128), with and without
    the normalisation (at that width the scaling is tensor operations; gradients of the normalised q, k as always)."""
    b, h, n, t = 2, 2, 400, 6.0
    q, k, v, go = (rnd(b, h, n, d, seed=s).bfloat16() for s in (80, 81, 82, 83))
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    o = sf.FASTMultiHeadAttention_Function.apply(qd, kd, vd, None, None, True, 0.0, normalize, t, 1.0, 1.0, 0.5, 1.5, 2)
    assert o.shape == (b, h, n, d) and o.dtype == torch.bfloat16
    o.backward(go.to(DEV))
    qr, kr, vr = (x.double().requires_grad_(True) for x in (q, k, v))
    if normalize:
        # the wrapper scales bf16 tensors by a bf16 factor: the same rounded factor here
        fq = (1.5 / q.float().norm(dim=-1).amax(dim=-1)[..., None, None]).bfloat16().double()
        fk = (1.5 / k.float().norm(dim=-1).amax(dim=-1)[..., None, None]).bfloat16().double()
        qn, kn = (qr * fq).bfloat16().double(), (kr * fk).bfloat16().double()
        qn.requires_grad_(True); kn.requires_grad_(True)
    else:
        qn, kn = qr, kr
    qn.retain_grad(); kn.retain_grad()
    oref, _ = O.closed_form_forward(qn, kn, vr, mask=True, tau=t, p=2)
    oref.backward(go.double())
    assert rel_err(o, oref) < TOL[torch.bfloat16]
    for got, want in ((qd.grad, qn.grad), (kd.grad, kn.grad), (vd.grad, vr.grad)):
        assert got.shape == want.shape and rel_err(got, want) < TOL[torch.bfloat16]
    with pytest.raises(RuntimeError, match="unsupported head size"):
        sf.FASTMultiHeadAttention_Function.apply(*(rnd(1, 1, 8, 130).bfloat16().to(DEV) for _ in range(3)))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 3, 333, 64), (5, 700, 32), (1, 1, 1, 64)])
def test_dormant_steps_kernels(dtype, shape):
    """fastmax_key_rpe / fastmax_output_noise through the C ABI against the oracle's restatement of the
    reference's switched-off steps (fastmax_cuda_forward.cu:282-292, :340-349), on packed tensors, on the
    projection layout and in place."""
    from reproducing_fastmax_results_amd._capi import get_lib
    lib = get_lib()
    n, d, t = shape[-2], shape[-1], 3.5
    k = rnd(*shape, seed=71).to(dtype)
    rpe = rnd(2 * n - 1, d, seed=72)
    want = O.apply_rpe_and_temp(k.double(), rpe, t) * t          # the pass leaves the division to the operator
    got = lib.key_rpe(k.to(DEV), rpe.to(DEV), t)
    assert rel_err(got, want) < (1e-6 if dtype == torch.float32 else 4e-3)
    noise = rnd(*shape, seed=73).to(dtype)
    want = O.apply_dropout(k.double(), noise.double(), 0.3)
    got = lib.output_noise(k.to(DEV), noise.to(DEV), 0.3)
    assert rel_err(got, want) < (1e-6 if dtype == torch.float32 else 4e-3)
    assert torch.equal(lib.output_noise(k.to(DEV), noise.to(DEV), 0.0).cpu(), k)
    if len(shape) == 4 and shape[1] > 1:
        # (b, n, h, d) memory seen as (b, h, n, d), written in place
        kp = k.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3)
        np_ = noise.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3)
        out = lib.output_noise(kp, np_, 0.3, out=kp)
        assert out.data_ptr() == kp.data_ptr()
        assert rel_err(kp, want) < (1e-6 if dtype == torch.float32 else 4e-3)


def test_dormant_steps_errors():
    from reproducing_fastmax_results_amd._capi import FastmaxError, get_lib
    lib = get_lib()
    k = torch.zeros(2, 10, 64, device=DEV)
    with pytest.raises(ValueError):
        lib.key_rpe(k, torch.zeros(20, 64, device=DEV), 1.0)          # 2n-1 = 19 rows
    with pytest.raises(FastmaxError):
        lib.key_rpe(k, torch.zeros(19, 64, device=DEV), 0.0)          # temperature must be positive
    with pytest.raises(ValueError):
        lib.output_noise(k, torch.zeros(2, 10, 64, device=DEV, dtype=torch.bfloat16), 0.1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d", [64, 48])
def test_operator_with_dormant_steps(sf, dtype, d):
    """The operator with key RPE and output noise on, gradients included, against the closed form on the
    keys and output the oracle's restatement of the two steps gives."""
    b, h, n, t, scale = 2, 2, 300, 6.0, 0.25
    q, k, v, go, noise = (rnd(b, h, n, d, seed=s).to(dtype) for s in (81, 82, 83, 84, 85))
    rpe = rnd(2 * n - 1, d, seed=86)
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    o = sf.fastmax_with_dormant_steps(qd, kd, vd, noise.to(DEV), rpe.to(DEV), mask=True, noise_scale=scale,
                                      rpe_on_keys=True, temperature=t, p=2)
    o.backward(go.to(DEV))
    q64, k64, v64 = (x.double().requires_grad_(True) for x in (q, k, v))
    keys = O.apply_rpe_and_temp(k64, rpe, t)                      # already divided by the temperature
    o64, _ = O.closed_form_forward(q64, keys, v64, mask=True, tau=1.0, p=2)
    o64 = O.apply_dropout(o64, noise, scale)
    o64.backward(go.double())
    assert rel_err(o, o64) < TOL[dtype]
    for got, want in ((qd.grad, q64.grad), (kd.grad, k64.grad), (vd.grad, v64.grad)):
        assert rel_err(got, want) < TOL[dtype]
    # both switched off: the plain operator
    o_plain = sf.fastmax_with_dormant_steps(qd, kd, vd, noise.to(DEV), rpe.to(DEV), mask=True, temperature=t, p=2)
    o_ref = sf.FASTMultiHeadAttention_Function.apply(qd, kd, vd, None, None, True, 0.0, False, t, 1.0, 1.0, 0.5, 1.0, 2)
    assert torch.equal(o_plain, o_ref)
