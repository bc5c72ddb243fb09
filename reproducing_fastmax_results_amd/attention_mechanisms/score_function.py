"""Operator fronts of the Fastmax path, on the HIP kernels.

Mirrors, name for name, what a model written against the reference imports:

* ``FASTMultiHeadAttention_Function`` / ``FASTMultiHeadAttention`` /
  ``rpe_matrix_creator`` / ``fastmax_custom`` - the autograd wrapper around the
  extension (reference ``transformer/model.py:14-74, 208-248``), same argument
  list ``(q, k, v, drop_noise, rpe_matrix, mask, dropout, normalize,
  temperature, a0, a1, a2, lim, p)``;
* ``fastmax(q, k, v, mask, denum_term, normalize, p, create_attn_matrix,
  dropout_rate)`` - the score function (reference
  ``attention_mechanisms/score_function.py:7-17``);
* ``fastmax_einops(q, k, v, mask, normalize_term, tensors_normalized, p, ...)`` -
  the einops front (reference ``attention_mechanisms/fastattention_einops.py:7-27``).

Differences from the reference wrapper, all deliberate:
the (b,h,n,d) <-> (n,b*h,d) transposes and their copies are gone (the kernels take
strides), nothing is mutated in place, and the gradient with respect to k carries
the 1/temperature factor inside the kernel instead of a separate division.
There is no fallback: without the built extension the import fails.
"""
from __future__ import annotations

import math

import torch

from .. import fastmax_cuda as _ext   # the torch binding built by __graft_entry__.build()

__all__ = [
    "FASTMultiHeadAttention_Function", "FASTMultiHeadAttention", "rpe_matrix_creator", "fastmax_custom",
    "fastmax", "fastmax_einops", "FastmaxNormalize", "FastmaxNormAttention", "FastmaxDecodeState",
    "FastmaxOutputNoise", "FastmaxKeyRpe", "fastmax_with_dormant_steps",
]

CENTRE_NONE, CENTRE_FEATURE, CENTRE_TOKEN = 0, 1, 2


_HEAD_SIZES = (32, 64)      # what every kernel is built for
_WIDE_HEAD = 128            # bf16 attention alone also runs at this width (dense tiles; no normalisation or decoding kernels)


def _pad_features(x, wide=False):
    """x itself, or a copy zero-padded along the feature axis to the next head size the kernels
    are built for.  Zero features change neither q.k nor any norm, padded value columns come out
    as zero output columns, and the padded columns of every gradient are zero as well, so callers
    pad on the way in and slice on the way out.  ``wide``: the caller's kernels also exist at 128
    (attention on bf16 tensors)."""
    d = x.shape[-1]
    sizes = _HEAD_SIZES + ((_WIDE_HEAD,) if wide and x.dtype == torch.bfloat16 else ())
    for size in sizes:
        if d == size:
            return x
        if d < size:
            return torch.nn.functional.pad(x, (0, size - d))
    raise RuntimeError(f"fastmax: unsupported head size {d} for {x.dtype} (the kernels cover up to {_HEAD_SIZES[-1]}, "
                       f"attention on bfloat16 tensors up to {_WIDE_HEAD})")


class FastmaxNormalize(torch.autograd.Function):
    """``y = scale * (x - centre) / max_n ||x_n - centre||_2`` per (b, h), forward and
    backward on the HIP passes.  The reference's extension drops this gradient; its
    Python variants carry it through autograd (``score_function.py:40-55``,
    ``fastattention_einops.py:327-334``), which the backward pass reproduces."""

    @staticmethod
    def forward(ctx, x, centre: int = CENTRE_NONE, scale: float = 1.0):
        d = x.shape[-1]
        if centre != CENTRE_FEATURE:            # the feature mean is the one thing padding would change
            x = _pad_features(x)
        ctx.save_for_backward(x)
        ctx.centre, ctx.scale, ctx.d = centre, scale, d
        return _ext.normalize(x, centre, True, scale)[..., :d]

    @staticmethod
    def backward(ctx, grad_y):
        (x,) = ctx.saved_tensors
        if x.shape[-1] != ctx.d:
            grad_y = _pad_features(grad_y)
        return _ext.normalize_backward(x, grad_y, ctx.centre, True, ctx.scale)[..., :ctx.d], None, None


def _fold_possible(q, k, mask):
    """The folded normalisation covers everything but causal attention with more keys than queries
    (two sub-problems would share one Jacobian); that case takes the separate normalisation pass."""
    return not (mask and k.shape[-2] > q.shape[-2])


class FastmaxNormAttention(torch.autograd.Function):
    """Fastmax attention on ``lim * x / max_n ||x_n||_2`` of q and k (per batch and head), the
    normalisation folded into the kernels: one statistics pass reads q and k once, the attention
    kernels scale the rows as they load them, and the backward returns the gradients with respect to
    the RAW q and k, the normalisation's own Jacobian included (the dQ / dK kernels scale what they
    store and one small kernel adds the rank-one term of the row with the largest norm).  Replaces the
    reference's ``apply_norm`` pass (``fastmax_cuda_forward.cu:326-338``) and the autograd graph of its
    Python variants (``score_function.py:40-55``); semantics of ``transformer/model.py:97-102``."""

    @staticmethod
    def forward(ctx, q, k, v, mask=False, lim=1.0, temperature=1.0, a0=1.0, a1=1.0, a2=0.5, p=2):
        d = q.shape[-1]
        q, k, v = _pad_features(q), _pad_features(k), _pad_features(v)
        qk, kk = _ext.maxnorm_stats(q, k)
        cfg = (bool(mask), 1.0 / float(temperature), float(a0), float(a1), float(a2), int(p))
        o, g, saved = _ext.forward_norm(q, k, v, qk, kk, float(lim), *cfg, 0, 0)
        if any(ctx.needs_input_grad[:3]):
            ctx.save_for_backward(q, k, v, o, g, saved, qk, kk)
        ctx.cfg, ctx.lim, ctx.d = cfg, float(lim), d
        return o[..., :d]

    @staticmethod
    def backward(ctx, grad_output):
        q, k, v, o, g, saved, qk, kk = ctx.saved_tensors
        if q.shape[-1] != ctx.d:
            grad_output = _pad_features(grad_output)
        gq, gk, gv = _ext.backward_norm(q, k, v, o, g, grad_output, saved, qk, kk, ctx.lim, True, *ctx.cfg, 0, 0)
        d = ctx.d
        return (gq[..., :d], gk[..., :d], gv[..., :d]) + (None,) * 7


class FastmaxOutputNoise(torch.autograd.Function):
    """``o * (1 + scale * noise)``: the reference's ``apply_dropout`` (``fastmax_cuda_forward.cu:340-349``),
    which its ``forward_cuda`` calls with scale 0 (``:443``).  The backward is the same pass on dO."""

    @staticmethod
    def forward(ctx, o, noise, scale):
        d = o.shape[-1]
        noise = _pad_features(noise.to(o.dtype))
        ctx.save_for_backward(noise)
        ctx.scale, ctx.d = float(scale), d
        return _ext.output_noise(_pad_features(o), noise, float(scale))[..., :d]

    @staticmethod
    def backward(ctx, grad_y):
        (noise,) = ctx.saved_tensors
        return _ext.output_noise(_pad_features(grad_y), noise, ctx.scale)[..., :ctx.d], None, None


class FastmaxKeyRpe(torch.autograd.Function):
    """``k + temperature * rpe[(l + n) % (2n - 1)]``: keys that make the operator see ``k / temperature +
    rpe``, the addition the reference leaves commented out (``fastmax_cuda_forward.cu:289``).  The gradient
    with respect to k passes through; the table gets none (the reference never trains through it)."""

    @staticmethod
    def forward(ctx, k, rpe, temperature):
        d = k.shape[-1]
        ctx.d = d
        kp = _pad_features(k)
        table = torch.nn.functional.pad(rpe, (0, kp.shape[-1] - d))
        return _ext.key_rpe(kp, table, float(temperature))[..., :d]

    @staticmethod
    def backward(ctx, grad_k):
        return grad_k, None, None


def fastmax_with_dormant_steps(q, k, v, drop_noise=None, rpe_matrix=None, mask=False, noise_scale=0.0, rpe_on_keys=False,
                               normalize=False, temperature=1.0, a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2):
    """The operator with the two steps switched on that the reference's ``forward_cuda`` carries switched off:
    ``rpe_on_keys`` adds ``rpe_matrix`` rows to ``k / temperature`` (``fastmax_cuda_forward.cu:289``) and a non-zero
    ``noise_scale`` multiplies the output by ``1 + noise_scale * drop_noise`` (``:340-349``).  With both off
    this is ``FASTMultiHeadAttention_Function.apply``; the order of the steps is the reference's
    (temperature and RPE, normalisation, attention, noise)."""
    if rpe_on_keys:
        if rpe_matrix is None:
            raise ValueError("rpe_on_keys needs rpe_matrix (rpe_matrix_creator)")
        k = FastmaxKeyRpe.apply(k, rpe_matrix, temperature)
    o = FASTMultiHeadAttention_Function.apply(q, k, v, None, None, mask, 0.0, normalize, temperature, a0, a1, a2, lim, p)
    if noise_scale:
        if drop_noise is None:
            raise ValueError("a non-zero noise_scale needs drop_noise")
        o = FastmaxOutputNoise.apply(o, drop_noise, noise_scale)
    return o


class FASTMultiHeadAttention_Function(torch.autograd.Function):
    """Same call as reference ``transformer/model.py:16``.  q, k, v: ``(b, h, n, d)`` or
    ``(b*h, n, d)``.  ``drop_noise``, ``rpe_matrix`` and ``dropout`` are accepted and unused,
    as in the reference extension (``fastmax_cuda_forward.cu:289, 443``).  With
    ``normalize`` the tensors are first mapped to ``lim * x / max_n ||x_n||`` (the
    semantics spelled out in ``transformer/model.py:97-102``) and, like the reference,
    the returned gradients are those with respect to the normalised q and k.  Head sizes other
    than 32 and 64 (up to 64; on bfloat16 tensors up to 128) run zero-padded to the next size the kernels have.
    """

    @staticmethod
    def forward(ctx, q, k, v, drop_noise=None, rpe_matrix=None, mask=False, dropout=0.0, normalize=False,
                temperature=1.0, a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2):
        if q.dim() not in (3, 4):
            raise ValueError("q, k, and v should be either 3 or 4 dimensional tensors. "
                             "If 3D: (b*h,n,d), if 4D: (b,h,n,d).")
        d = q.shape[-1]
        q, k, v = _pad_features(q, True), _pad_features(k, True), _pad_features(v, True)
        inv_tau = 1.0 / float(temperature)
        ctx.fold = None
        if normalize and q.shape[-1] > _HEAD_SIZES[-1]:
            # no normalisation kernels at that width: the scaling itself (lim * x / max_n ||x_n||, transformer/model.py:97-102)
            # as tensor operations; like the reference, the gradients returned are those of the normalised q and k
            q = q * (float(lim) / q.float().norm(dim=-1).amax(dim=-1)[..., None, None]).to(q.dtype)
            k = k * (float(lim) / k.float().norm(dim=-1).amax(dim=-1)[..., None, None]).to(k.dtype)
            normalize = False
        if normalize and _fold_possible(q, k, mask):
            # normalised on load; like the reference, the backward returns the gradients with respect to the
            # normalised q and k (its extension has no backward of apply_norm)
            qk, kk = _ext.maxnorm_stats(q, k)
            o, g, saved = _ext.forward_norm(q, k, v, qk, kk, float(lim), bool(mask), inv_tau, float(a0), float(a1),
                                            float(a2), int(p), 0, 0)
            if any(ctx.needs_input_grad[:3]):
                ctx.save_for_backward(q, k, v, o, g, saved, qk, kk)
            ctx.fold = float(lim)
            ctx.cfg = (bool(mask), inv_tau, float(a0), float(a1), float(a2), int(p), d)
            return o[..., :d]
        if normalize:
            q = _ext.normalize(q, CENTRE_NONE, True, float(lim))
            k = _ext.normalize(k, CENTRE_NONE, True, float(lim))
        needs_grad = any(ctx.needs_input_grad[:3])
        if needs_grad:
            # keep the key-side copies and prefix states the forward built: the backward reuses them
            o, g, saved = _ext.forward_save(q, k, v, bool(mask), inv_tau, float(a0), float(a1), float(a2), int(p), 0, 0)
            ctx.save_for_backward(q, k, v, o, g, saved)
        else:
            o, g = _ext.forward_ex(q, k, v, bool(mask), inv_tau, float(a0), float(a1), float(a2), int(p), 0, 0)
        ctx.cfg = (bool(mask), inv_tau, float(a0), float(a1), float(a2), int(p), d)
        return o[..., :d]

    @staticmethod
    def backward(ctx, grad_output):
        mask, inv_tau, a0, a1, a2, p, d = ctx.cfg
        if ctx.fold is not None:
            q, k, v, o, g, saved, qk, kk = ctx.saved_tensors
            if q.shape[-1] != d:
                grad_output = _pad_features(grad_output)
            gq, gk, gv = _ext.backward_norm(q, k, v, o, g, grad_output, saved, qk, kk, ctx.fold, False, mask, inv_tau,
                                            a0, a1, a2, p, 0, 0)
            return (gq[..., :d], gk[..., :d], gv[..., :d]) + (None,) * 11
        q, k, v, o, g, saved = ctx.saved_tensors
        if q.shape[-1] != d:
            grad_output = _pad_features(grad_output, True)
        gq, gk, gv = _ext.backward_saved(q, k, v, o, g, grad_output, saved, mask, inv_tau, a0, a1, a2, p, 0, 0)
        return (gq[..., :d], gk[..., :d], gv[..., :d]) + (None,) * 11


class FastmaxDecodeState:
    """The persistent moment state of incremental decoding for one attention layer: the sums the
    reference's causal kernel runs along the sequence (``fastmax_cuda_forward.cu:160-276``), kept between
    calls, so that a generation step costs the same whatever the number of tokens before it (the
    reference's loop, ``transformer/eval.py:8-32``, runs the whole context for every token).
    ``prompt(q, k, v)``: ordinary causal attention over a first block of tokens, whose keys and values are
    then absorbed; ``step(q, k, v)``: one token.  Tensors are ``(b, h, n, d)`` or ``(b*h, n, d)``; no
    gradients; q and k unnormalised (the max-norm depends on every token)."""

    def __init__(self, temperature=1.0, a0=1.0, a1=1.0, a2=0.5, p=2):
        self.args = (1.0 / float(temperature), float(a0), float(a1), float(a2), int(p))
        self.state, self.tokens = None, 0

    def _absorb(self, k, v):
        if self.state is None:
            self.state = _ext.decode_state(k, *self.args)
        _ext.decode_absorb(k, v, self.state, *self.args)
        self.tokens += k.shape[-2]

    @torch.no_grad()
    def prompt(self, q, k, v):
        if self.tokens:
            raise ValueError("the state takes a block of tokens only while it is empty; then single tokens")
        d = q.shape[-1]
        q, k, v = _pad_features(q), _pad_features(k), _pad_features(v)
        inv_tau, a0, a1, a2, p = self.args
        o, _ = _ext.forward_ex(q, k, v, True, inv_tau, a0, a1, a2, p, 0, 0)
        self._absorb(k, v)
        return o[..., :d]

    @torch.no_grad()
    def step(self, q, k, v):
        d = q.shape[-1]
        q, k, v = _pad_features(q), _pad_features(k), _pad_features(v)
        if self.state is None:
            self.state = _ext.decode_state(k, *self.args)
        o, _ = _ext.decode_step(q, k, v, self.state, *self.args)
        self.tokens += 1
        return o[..., :d]


def fastmax_function(q, k, v, mask=0, dropout_rate=0.0, normalize=0, temperature=1, a0=1, a1=1, a2=0.5, lim=1, p=2):
    """Functional form with the argument order of the reference's (disabled) pure-torch
    twin ``fastmax_function`` (``transformer/model.py:77``); routed to the kernels."""
    return FASTMultiHeadAttention_Function.apply(q, k, v, None, None, bool(mask), dropout_rate, bool(normalize),
                                                 temperature, a0, a1, a2, lim, p)


class FASTMultiHeadAttention(torch.nn.Module):
    """Reference ``transformer/model.py:208-216``."""

    def __init__(self, use_custom_gradient=True):
        super().__init__()
        self.use_custom_gradient = use_custom_gradient

    def forward(self, q, k, v, drop_noise=None, rpe_matrix=None, mask=False, dropout=0.0, normalize=False,
                temperature=1.0, a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2):
        return FASTMultiHeadAttention_Function.apply(q, k, v, drop_noise, rpe_matrix, mask, dropout, normalize,
                                                     temperature, a0, a1, a2, lim, p)


def rpe_matrix_creator(n, d, device, dtype, structured=False, is_zero=True):
    """``(2n-1, d)`` relative-position matrix (reference ``transformer/model.py:218-247``).
    The kernels do not read it (neither does the reference extension); it exists so
    that call sites written for the reference keep working."""
    if structured:
        position = torch.arange(0, n, device=device, dtype=dtype).unsqueeze(1)
        div_term = torch.exp(torch.arange(0, d, 2, device=device, dtype=dtype) * -(math.log(10000.0) / d))
        pos = torch.zeros(n, d, device=device, dtype=dtype)
        neg = torch.zeros(n, d, device=device, dtype=dtype)
        pos[:, 0::2] = torch.sin(position * div_term)
        pos[:, 1::2] = torch.cos(position * div_term)
        neg[:, 0::2] = torch.sin(-position * div_term)
        neg[:, 1::2] = torch.cos(-position * div_term)
        return torch.cat([torch.flip(pos, [0]), neg[1:]], dim=0)
    if is_zero:
        return torch.zeros(size=(2 * n - 1, d), device=device, dtype=dtype)
    return torch.normal(0, 1, size=(2 * n - 1, d), device=device, dtype=dtype)


fastmax_custom = FASTMultiHeadAttention()


def _attn_matrix(q, k, mask, tau, p):
    """Quadratic debug path (reference ``score_function.py:226-247``): explicit attention
    matrix in torch; not a hot path.  ``mask`` is what the reference takes there, a tensor
    broadcastable to ``(b, h, nq, nk)`` whose zero entries are removed
    (``torch.where(mask == 0, 0, attn)``, ``:243-244``); ``True`` is accepted as a shorthand
    for the lower-triangular mask, ``None`` / ``False`` remove nothing."""
    s = torch.matmul(q.float(), k.float().transpose(-1, -2)) / tau
    f = 1 + s + (0.5 * s * s if p == 2 else 0)
    if torch.is_tensor(mask):
        f = torch.where(mask.to(f.device) == 0, torch.zeros((), dtype=f.dtype, device=f.device), f)
    elif mask:
        f = f * torch.ones_like(f).tril()
    return f / f.sum(-1, keepdim=True)


def fastmax(q, k, v, mask=None, denum_term=8, normalize=0, p=1, create_attn_matrix=False, dropout_rate=0):
    """Same call as reference ``attention_mechanisms/score_function.py:7``.

    ``normalize == 1``: q and k are centred over tokens and divided by their largest
    token norm, and the score is their plain dot product; otherwise the score is
    divided by ``denum_term * sqrt(d)``.  ``dropout_rate`` must be 0 (the reference's
    random feature dropout has no seeded counterpart)."""
    if dropout_rate:
        raise NotImplementedError("fastmax: dropout_rate != 0 is not supported by the HIP path")
    d = q.shape[-1]
    if create_attn_matrix:
        a = _attn_matrix(q, k, mask, denum_term * math.sqrt(d), 2)
        return torch.matmul(a, v.float()).to(q.dtype), a
    masked = False if mask is None else bool(mask)      # reference: `if mask is None or not mask` -> unmasked
    if normalize == 1:
        q = FastmaxNormalize.apply(q, CENTRE_TOKEN, 1.0)
        k = FastmaxNormalize.apply(k, CENTRE_TOKEN, 1.0)
        temperature = 1.0
    else:
        temperature = denum_term * math.sqrt(d)
    return FASTMultiHeadAttention_Function.apply(q, k, v, None, None, masked, 0.0, False, temperature,
                                                 1.0, 1.0, 0.5, 1.0, int(p))


def fastmax_einops(q, k, v, mask=True, normalize_term=8, tensors_normalized=False, p=1, dropout_rate=0.0,
                   create_attn=False):
    """Same call as the reference's einops front (``fastattention_einops.py:7-27``): the
    score is divided by ``normalize_term * sqrt(d)`` unless ``tensors_normalized``
    (``:78-82``); ``mask`` follows the reference's identity test, anything but ``False``
    means causal (``:85``)."""
    d = q.shape[-1]
    tau = 1.0 if tensors_normalized is True else normalize_term * math.sqrt(d)
    masked = mask is not False
    if create_attn:
        a = _attn_matrix(q, k, masked, tau, int(p))
        return torch.matmul(a, v.float()).to(q.dtype), a
    return FASTMultiHeadAttention_Function.apply(q, k, v, None, None, masked, 0.0, False, tau, 1.0, 1.0, 0.5, 1.0, int(p))
