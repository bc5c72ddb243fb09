"""Shared helpers of the parity tests: seeded inputs and comparison with the oracle."""
import math

import torch

from oracle import fastmax_oracle as O

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}   # rel-L2 bars: fp32 1e-5, bf16 2e-2


def make_inputs(bh, nq, nk, d, dtype, device, seed=0, scale=1.0, go_scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    q = (scale * torch.randn(bh, nq, d, generator=gen)).to(dtype)
    k = (scale * torch.randn(bh, nk, d, generator=gen)).to(dtype)
    v = (scale * torch.randn(bh, nk, d, generator=gen)).to(dtype)
    go = (go_scale * torch.randn(bh, nq, d, generator=gen)).to(dtype)
    return tuple(t.to(device) for t in (q, k, v, go))


def rel_err(x, ref, cancel=None):
    """Plain rel-L2 ||x - ref|| / ||ref||, with no floor.

    ``cancel`` is only for a reference that is zero because two terms cancel exactly (dq, dk of a
    single causal token: gh.v and c are the same number): it is the per-element size of the terms that
    cancel, derived from the inputs by the caller (``cancel_scale``).  Only when ||ref|| is below 1e-9 of
    that size (the fp64 oracle's own rounding residue) is the error measured against it instead."""
    x = x.detach().double().cpu(); ref = ref.detach().double().cpu()
    den = float(ref.norm())
    if cancel is not None and den < 1e-9 * cancel * ref.numel() ** 0.5:
        den = cancel * ref.numel() ** 0.5
    if den == 0.0:
        return 0.0 if float((x - ref).norm()) == 0.0 else float("inf")
    return float((x - ref).norm() / den)


def cancel_scale(q, k, v, go, g, tau, a):
    """Per-element size of one of the terms whose difference is dq or dk: f'(s) (dO/g . v) k / tau, from the
    inputs' root-mean-squares (the scores' term with their rms)."""
    rms = lambda t: float(t.detach().double().pow(2).mean().sqrt())
    d = q.shape[-1]
    s = rms(q) * rms(k) * d ** 0.5 / tau
    gmin = max(float(g.detach().double().abs().min()), 1e-300)
    return (abs(a[1]) + 2 * abs(a[2]) * s) * rms(go) * rms(v) * d ** 0.5 * max(rms(q), rms(k)) / (tau * gmin)


def oracle_all(q, k, v, go, *, mask, tau, p, a=(1.0, 1.0, 0.5), block=1024):
    """fp64 closed form on the (already rounded) inputs: o, g, dq, dk, dv."""
    args = [t.detach().cpu().double() for t in (q, k, v, go)]
    if mask or q.shape[1] * k.shape[1] > 1 << 22:
        return O.manual_backward_blocked(*args, mask=mask, tau=tau, p=p, a0=a[0], a1=a[1], a2=a[2], block=block)
    return O.closed_form_forward_backward(*args, mask=mask, tau=tau, p=p, a0=a[0], a1=a[1], a2=a[2])


def check_forward(lib, bh, nq, d, dtype, device, *, mask, p, nk=None, chunk=0, flags=0, tau_mult=8.0,
                  a=(1.0, 1.0, 0.5), seed=0, scale=1.0):
    nk = nk or nq
    q, k, v, go = make_inputs(bh, nq, nk, d, dtype, device, seed, scale)
    tau = tau_mult * math.sqrt(d)
    o, g = lib.forward(q, k, v, mask=mask, inv_tau=1.0 / tau, a0=a[0], a1=a[1], a2=a[2], p=p, chunk=chunk, flags=flags)
    ref = oracle_all(q, k, v, go, mask=mask, tau=tau, p=p, a=a)
    eo, eg = rel_err(o, ref[0]), rel_err(g, ref[1])
    assert eo < TOL[dtype], f"o rel-L2 {eo:.3e}"
    assert eg < TOL[dtype], f"g rel-L2 {eg:.3e}"
    return eo, eg


def check_forward_backward(lib, bh, nq, d, dtype, device, *, mask, p, nk=None, chunk=0, flags=0, tau_mult=8.0,
                           a=(1.0, 1.0, 0.5), seed=0, scale=1.0, saved=False, go_scale=1.0):
    """saved: run the backward on the workspace the forward leaves behind
    (FASTMAX_FLAG_SAVE_FOR_BACKWARD / fastmax_backward_saved).  go_scale: size of the upstream gradient."""
    nk = nk or nq
    q, k, v, go = make_inputs(bh, nq, nk, d, dtype, device, seed, scale, go_scale)
    tau = tau_mult * math.sqrt(d)
    kw = dict(mask=mask, inv_tau=1.0 / tau, a0=a[0], a1=a[1], a2=a[2], p=p, chunk=chunk, flags=flags)
    if saved:
        o, g, ws = lib.forward(q, k, v, save=True, **kw)
        dq, dk, dv = lib.backward(q, k, v, o, g, go, saved=ws, **kw)
    else:
        o, g = lib.forward(q, k, v, **kw)
        dq, dk, dv = lib.backward(q, k, v, o, g, go, **kw)
    ref = oracle_all(q, k, v, go, mask=mask, tau=tau, p=p, a=a)
    cs = cancel_scale(q, k, v, go, ref[1], tau, a)
    errs = {n: rel_err(x, r, cs if n in ("dq", "dk") else None)
            for n, x, r in zip(("o", "g", "dq", "dk", "dv"), (o, g, dq, dk, dv), ref)}
    for n, e in errs.items():
        assert e < TOL[dtype], f"{n} rel-L2 {e:.3e} (all: {errs})"
    return errs


def check_batch_head_strides(lib, b, h, n, d, dtype, device, *, mask, p, chunk=0, seed=0):
    """q, k, v, dO as transposed views of (b, n, h*d) tensors, handed over with batch and head
    strides (FastmaxStrides.heads > 1), outputs written into the same memory order: bit-identical
    to the run on contiguous (b*h, n, d) copies."""
    gen = torch.Generator().manual_seed(seed)
    base = [torch.randn(b, n, h * d, generator=gen).to(dtype).to(device) for _ in range(4)]
    q4, k4, v4, go4 = (x.view(b, n, h, d).transpose(1, 2) for x in base)
    tau = 8.0 * math.sqrt(d)
    kw = dict(mask=mask, inv_tau=1.0 / tau, p=p, chunk=chunk)
    out = torch.empty(b, n, h, d, dtype=dtype, device=device).transpose(1, 2)
    o4, g4, ws = lib.forward(q4, k4, v4, save=True, out=out, **kw)
    q3, k3, v3, go3 = (x.contiguous().view(b * h, n, d) for x in (q4, k4, v4, go4))
    o3, g3, ws3 = lib.forward(q3, k3, v3, save=True, **kw)
    assert torch.equal(o4.contiguous().view(b * h, n, d), o3) and torch.equal(g4.reshape(b * h, n), g3)
    d4 = lib.backward(q4, k4, v4, o4, g4, go4, saved=ws, **kw)
    d3 = lib.backward(q3, k3, v3, o3, g3, go3, saved=ws3, **kw)
    for x4, x3 in zip(d4, d3):
        assert torch.equal(x4.contiguous().view(b * h, n, d), x3)
    return True


def check_norm_fold(lib, bh, nq, d, dtype, device, *, mask, p, nk=None, chunk=0, lim=1.5, tau=1.0, seed=0, saved=True,
                    jacobian=True, scale=1.0):
    """The max-norm normalisation of q and k folded into the kernels (FastmaxNormFold) against the fp64 closed
    form on lim * x / max_n ||x_n||: o, g, and either the gradients with respect to the raw q and k (torch
    autograd through the normalisation: ``jacobian``) or those with respect to the normalised tensors (what the
    reference's extension returns)."""
    nk = nk or nq
    q, k, v, go = make_inputs(bh, nq, nk, d, dtype, device, seed, scale)
    qk, kk = lib.maxnorm_stats(q, k)
    kw = dict(mask=mask, inv_tau=1.0 / tau, p=p, chunk=chunk, norm=(qk, kk, lim, jacobian))
    if saved:
        o, g, ws = lib.forward(q, k, v, save=True, **kw)
        dq, dk, dv = lib.backward(q, k, v, o, g, go, saved=ws, **kw)
    else:
        o, g = lib.forward(q, k, v, **kw)
        dq, dk, dv = lib.backward(q, k, v, o, g, go, **kw)
    qd, kd, vd, gd = (t.detach().cpu().double() for t in (q, k, v, go))
    if jacobian:
        qd.requires_grad_(True); kd.requires_grad_(True); vd.requires_grad_(True)
        oo, gg = O.closed_form_forward(O.normalize_lim(qd, lim), O.normalize_lim(kd, lim), vd, mask=mask, tau=tau, p=p)
        rq, rk, rv = torch.autograd.grad(oo, (qd, kd, vd), gd)
        ref = (oo.detach(), gg.detach(), rq, rk, rv)
    else:
        ref = oracle_all(O.normalize_lim(qd, lim), O.normalize_lim(kd, lim), vd, gd, mask=mask, tau=tau, p=p)
    errs = {n: rel_err(x, r) for n, x, r in zip(("o", "g", "dq", "dk", "dv"), (o, g, dq, dk, dv), ref)}
    for n, e in errs.items():
        assert e < TOL[dtype], f"{n} rel-L2 {e:.3e} (all: {errs})"
    return errs


def check_decode(lib, bh, n, n0, d, dtype, device, *, p, tau_mult=8.0, a=(1.0, 1.0, 0.5), seed=0, four_d=False):
    """Incremental decoding on the persistent moment state: the first n0 tokens are absorbed as a prompt, the
    others go through one step each; every step's o and g against the fp64 closed form of causal attention over
    the whole sequence (the state is fp32, so the bar is the fp32 one for fp32 tensors, the bf16 one for bf16)."""
    q, k, v, _ = make_inputs(bh, n, n, d, dtype, device, seed)
    tau = tau_mult * math.sqrt(d)
    kw = dict(inv_tau=1.0 / tau, p=p, a0=a[0], a1=a[1], a2=a[2])
    if four_d:                                   # (b, h, n, d) views of a (b, n, h*d) layout, two heads per batch
        assert bh % 2 == 0
        q, k, v = (t.view(bh // 2, 2, n, d).transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))
    state = lib.decode_state(k, **kw)
    if n0:
        lib.decode_absorb(k[..., :n0, :], v[..., :n0, :], state, **kw)
    outs, gs = [], []
    for t in range(n0, n):
        o, g = lib.decode_step(q[..., t:t + 1, :], k[..., t:t + 1, :], v[..., t:t + 1, :], state, **kw)
        outs.append(o); gs.append(g)
    o = torch.cat(outs, dim=-2).reshape(bh, n - n0, d)
    g = torch.cat(gs, dim=-1).reshape(bh, n - n0)
    q3, k3, v3 = (t.reshape(bh, n, d).detach().cpu().double() for t in (q, k, v))
    ro, rg = O.closed_form_forward(q3, k3, v3, mask=True, tau=tau, p=p, a0=a[0], a1=a[1], a2=a[2])
    eo, eg = rel_err(o, ro[:, n0:]), rel_err(g, rg[:, n0:])
    assert eo < TOL[dtype] and eg < TOL[dtype], f"decode o {eo:.3e} g {eg:.3e}"
    return eo, eg
