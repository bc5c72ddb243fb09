"""ctypes view of the C ABI declared in ``include/fastmax_hip.h``.

This is plumbing: it turns torch tensors into (pointer, strides) pairs, asks the
library how much scratch a call needs, allocates it with torch and passes torch's
current HIP stream.  There is no fallback: if ``libfastmax_hip.so`` has not been
built, importing the operator fails with an ImportError that says so.
"""
from __future__ import annotations

import ctypes as C
import os
import threading
from typing import Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libfastmax_hip.so"
# The same sources built with -DFM_BENCH_AIDS: per-kernel event timing and two matrix-rate yardsticks on top
# of the product's entry points.  Only bench.py and the tests of those aids load it.
BENCH_LIB_NAME = "libfastmax_hip_bench.so"

F32, BF16 = 0, 1
FLAG_FORCE_MOMENTS, FLAG_FORCE_DENSE, FLAG_SAVE_FOR_BACKWARD, FLAG_F32_COMPUTE = 1, 2, 4, 8
STATUS_OK = 0


class Strides(C.Structure):
    """FastmaxStrides: one stride for the batch*head axis, or batch and head strides (heads > 1)."""
    _fields_ = [("bh", C.c_int64), ("n", C.c_int64), ("b", C.c_int64), ("heads", C.c_int32), ("reserved", C.c_int32)]

    def __init__(self, bh=0, n=0, b=0, heads=0):
        super().__init__(bh, n, b, heads, 0)


class NormFold(C.Structure):
    """FastmaxNormFold: max-norm normalisation of q and k folded into the kernels' loads."""
    _fields_ = [("q_keys", C.c_void_p), ("k_keys", C.c_void_p), ("lim", C.c_float), ("grad", C.c_int32)]


class Desc(C.Structure):
    _fields_ = [
        ("bh", C.c_int32), ("nq", C.c_int32), ("nk", C.c_int32), ("d", C.c_int32),
        ("dtype", C.c_int32), ("mask", C.c_int32), ("p", C.c_int32),
        ("a0", C.c_float), ("a1", C.c_float), ("a2", C.c_float), ("inv_tau", C.c_float),
        ("chunk", C.c_int32), ("flags", C.c_int32),
        ("sq", Strides), ("sk", Strides), ("sv", Strides), ("so", Strides), ("sg", Strides),
        ("sdo", Strides), ("sdq", Strides), ("sdk", Strides), ("sdv", Strides),
        ("norm", NormFold),
    ]


class NormDesc(C.Structure):
    _fields_ = [
        ("bh", C.c_int32), ("n", C.c_int32), ("d", C.c_int32), ("dtype", C.c_int32),
        ("centre", C.c_int32), ("max_norm", C.c_int32), ("scale", C.c_float),
        ("sx", Strides), ("sy", Strides),
    ]


EXPORTS = (
    "fastmax_workspace_bytes", "fastmax_forward", "fastmax_backward", "fastmax_backward_saved", "fastmax_normalize",
    "fastmax_normalize_stats_bytes", "fastmax_normalize_backward", "fastmax_normalize_backward_stats_bytes",
    "fastmax_status_string", "fastmax_version", "fastmax_probe_mfma", "fastmax_probe_lds_transpose",
    "fastmax_key_rpe", "fastmax_output_noise", "fastmax_forward_static",
    "fastmax_maxnorm_stats", "fastmax_maxnorm_stats_bytes",
    "fastmax_decode_state_bytes", "fastmax_decode_scratch_bytes", "fastmax_decode_absorb", "fastmax_decode_step",
)
BENCH_EXPORTS = ("fastmax_profile_begin", "fastmax_profile_end", "fastmax_probe_mfma_rate", "fastmax_probe_mix_rate")
STATIC_SCRATCH_BYTES = 64 << 20     # FASTMAX_STATIC_SCRATCH_BYTES


class FastmaxError(RuntimeError):
    pass


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise FastmaxError(f"fastmax: dtype must be float32 or bfloat16, got {t.dtype}")


def _strides(t: torch.Tensor) -> Strides:
    """(bh, n, d) view: one stride for the batch*head axis; (b, h, n, d) view: batch and head strides,
    so the transposed view of a (b, n, h*d) projection output is taken as it is."""
    if t.dim() not in (3, 4):
        raise FastmaxError("fastmax: expected a (bh, n, d) or (b, h, n, d) view")
    if t.shape[-1] > 1 and t.stride(-1) != 1:
        raise FastmaxError("fastmax: the feature axis must be contiguous")
    if t.dim() == 3:
        return Strides(t.stride(0), t.stride(1))
    if t.shape[1] == 1:
        # one head per batch: the batch stride is the stride of the whole axis (stride(1) of such a view is
        # arbitrary: d for the transposed (b, n, 1, d) projection layout)
        return Strides(t.stride(0), t.stride(2))
    return Strides(t.stride(1), t.stride(2), t.stride(0), t.shape[1])


def _dims(t: torch.Tensor):
    """(batch*heads, tokens, features) of a 3-D or 4-D view."""
    if t.dim() == 4:
        return t.shape[0] * t.shape[1], t.shape[2], t.shape[3]
    return tuple(t.shape)


def _gstrides(g: torch.Tensor) -> Strides:
    """Strides of the denominators: (bh, n) or (b, h, n)."""
    if g.dim() == 3 and g.shape[1] == 1:
        return Strides(g.stride(0), g.stride(2))
    if g.dim() == 3:
        return Strides(g.stride(1), g.stride(2), g.stride(0), g.shape[1])
    return Strides(g.stride(0), g.stride(1))


class FastmaxLib:
    """One loaded copy of the shared library."""

    def __init__(self, path: Optional[str] = None, bench: bool = False):
        path = path or os.path.join(_HERE, BENCH_LIB_NAME if bench else LIB_NAME)
        self.bench = bench
        if not os.path.exists(path):
            raise ImportError(
                f"{path} not found: build it with `python __graft_entry__.py` "
                "(hipcc --offload-arch=gfx950); there is no CPU fallback")
        self.path = path
        self.lib = C.CDLL(path)
        L = self.lib
        L.fastmax_workspace_bytes.argtypes = [C.POINTER(Desc), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
        L.fastmax_workspace_bytes.restype = C.c_int
        L.fastmax_forward.argtypes = [C.POINTER(Desc)] + [C.c_void_p] * 6 + [C.c_size_t, C.c_void_p]
        L.fastmax_forward.restype = C.c_int
        L.fastmax_forward_static.argtypes = [C.POINTER(Desc)] + [C.c_void_p] * 6
        L.fastmax_forward_static.restype = C.c_int
        L.fastmax_backward.argtypes = [C.POINTER(Desc)] + [C.c_void_p] * 10 + [C.c_size_t, C.c_void_p]
        L.fastmax_backward.restype = C.c_int
        L.fastmax_backward_saved.argtypes = [C.POINTER(Desc)] + [C.c_void_p] * 10 + [C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]
        L.fastmax_backward_saved.restype = C.c_int
        L.fastmax_normalize.argtypes = [C.POINTER(NormDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.fastmax_normalize.restype = C.c_int
        L.fastmax_normalize_stats_bytes.argtypes = [C.POINTER(NormDesc)]
        L.fastmax_normalize_stats_bytes.restype = C.c_size_t
        L.fastmax_normalize_backward.argtypes = [C.POINTER(NormDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                                 C.c_void_p]
        L.fastmax_normalize_backward.restype = C.c_int
        L.fastmax_normalize_backward_stats_bytes.argtypes = [C.POINTER(NormDesc)]
        L.fastmax_normalize_backward_stats_bytes.restype = C.c_size_t
        L.fastmax_maxnorm_stats_bytes.argtypes = [C.c_int32, C.c_int32]
        L.fastmax_maxnorm_stats_bytes.restype = C.c_size_t
        L.fastmax_maxnorm_stats.argtypes = [C.POINTER(NormDesc), C.c_void_p, C.c_void_p, C.POINTER(NormDesc), C.c_void_p,
                                            C.c_void_p, C.c_void_p]
        L.fastmax_maxnorm_stats.restype = C.c_int
        for fn in (L.fastmax_decode_state_bytes, L.fastmax_decode_scratch_bytes):
            fn.argtypes = [C.POINTER(Desc)]
            fn.restype = C.c_size_t
        L.fastmax_decode_absorb.argtypes = [C.POINTER(Desc)] + [C.c_void_p] * 4
        L.fastmax_decode_absorb.restype = C.c_int
        L.fastmax_decode_step.argtypes = [C.POINTER(Desc)] + [C.c_void_p] * 8
        L.fastmax_decode_step.restype = C.c_int
        L.fastmax_status_string.argtypes = [C.c_int]
        L.fastmax_status_string.restype = C.c_char_p
        L.fastmax_version.restype = C.c_int
        L.fastmax_probe_mfma.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.fastmax_probe_mfma.restype = C.c_int
        L.fastmax_probe_lds_transpose.argtypes = [C.c_void_p, C.c_void_p]
        L.fastmax_probe_lds_transpose.restype = C.c_int
        L.fastmax_key_rpe.argtypes = [C.POINTER(NormDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p]
        L.fastmax_key_rpe.restype = C.c_int
        L.fastmax_output_noise.argtypes = [C.POINTER(NormDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p]
        L.fastmax_output_noise.restype = C.c_int
        if bench:
            L.fastmax_probe_mfma_rate.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p]
            L.fastmax_probe_mfma_rate.restype = C.c_int
            L.fastmax_probe_mix_rate.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
            L.fastmax_probe_mix_rate.restype = C.c_int
            L.fastmax_profile_begin.restype = C.c_int
            L.fastmax_profile_end.argtypes = [C.POINTER(C.c_int), C.POINTER(C.c_float), C.c_int]
            L.fastmax_profile_end.restype = C.c_int

    # -- helpers ---------------------------------------------------------------
    def status_string(self, st: int) -> str:
        return self.lib.fastmax_status_string(st).decode()

    def check(self, st: int, what: str) -> None:
        if st != STATUS_OK:
            raise FastmaxError(f"{what}: {self.status_string(st)} (status {st})")

    @staticmethod
    def _stream(t: torch.Tensor) -> int:
        if t.is_cuda:
            return torch.cuda.current_stream(t.device).cuda_stream
        return 0

    def maxnorm_stats(self, q, k=None):
        """Statistics of the folded max-norm normalisation (fastmax_maxnorm_stats): one int64 tensor
        (bh, blocks of 256 tokens) per given tensor, q and k in one launch."""
        descs, keys = [], []
        for t in (q, k):
            if t is None:
                continue
            nd = NormDesc()
            nd.bh, nd.n, nd.d = _dims(t)
            nd.dtype, nd.sx = _dtype_code(t), _strides(t)
            descs.append(nd)
            nbytes = self.lib.fastmax_maxnorm_stats_bytes(nd.bh, nd.n)
            keys.append(torch.empty(nd.bh, nbytes // 8 // nd.bh, dtype=torch.int64, device=t.device))
        if k is None:
            st = self.lib.fastmax_maxnorm_stats(C.byref(descs[0]), q.data_ptr(), keys[0].data_ptr(), None, None, None,
                                                self._stream(q))
        else:
            st = self.lib.fastmax_maxnorm_stats(C.byref(descs[0]), q.data_ptr(), keys[0].data_ptr(), C.byref(descs[1]),
                                                k.data_ptr(), keys[1].data_ptr(), self._stream(q))
        self.check(st, "fastmax_maxnorm_stats")
        return keys[0] if k is None else tuple(keys)

    def make_desc(self, q, k, v, *, mask, inv_tau, a0, a1, a2, p, chunk=0, flags=0, norm=None) -> Desc:
        d = Desc()
        d.bh, d.nq, d.d = _dims(q)
        kb, d.nk, kd = _dims(k)
        if kb != d.bh or kd != d.d or _dims(v) != (d.bh, d.nk, d.d):
            raise FastmaxError("fastmax: q, k, v must be (bh, nq, d), (bh, nk, d), (bh, nk, d)")
        d.dtype = _dtype_code(q)
        if k.dtype != q.dtype or v.dtype != q.dtype:
            raise FastmaxError("fastmax: q, k, v must share one dtype")
        d.mask, d.p = int(bool(mask)), int(p)
        d.a0, d.a1, d.a2, d.inv_tau = float(a0), float(a1), float(a2), float(inv_tau)
        d.chunk, d.flags = int(chunk), int(flags)
        d.sq, d.sk, d.sv = _strides(q), _strides(k), _strides(v)
        if norm is not None:
            # (q_keys, k_keys, lim, grad): tensors from maxnorm_stats (or None), see FastmaxNormFold
            qk, kk, lim, grad = norm
            d.norm.q_keys = qk.data_ptr() if qk is not None else None
            d.norm.k_keys = kk.data_ptr() if kk is not None else None
            d.norm.lim, d.norm.grad = float(lim), int(bool(grad))
        return d

    def workspace_bytes(self, desc: Desc) -> Tuple[int, int]:
        f, b = C.c_size_t(0), C.c_size_t(0)
        self.check(self.lib.fastmax_workspace_bytes(C.byref(desc), C.byref(f), C.byref(b)), "fastmax_workspace_bytes")
        return f.value, b.value

    @staticmethod
    def _workspace(nbytes: int, device) -> torch.Tensor:
        # torch allocations are at least 256-byte aligned on the device; on the CPU
        # (host simulator) over-allocate and slice to an aligned start
        buf = torch.empty(nbytes + 256, dtype=torch.uint8, device=device)
        off = (-buf.data_ptr()) % 256
        return buf[off:off + nbytes]

    # -- entry points ------------------------------------------------------------
    def forward(self, q, k, v, *, mask, inv_tau, a0=1.0, a1=1.0, a2=0.5, p=2, chunk=0, flags=0,
                out: Optional[torch.Tensor] = None, g: Optional[torch.Tensor] = None, save: bool = False,
                ws: Optional[torch.Tensor] = None, norm=None):
        """q (bh, nq, d), k, v (bh, nk, d) views with contiguous features, or (b, h, n, d) views.
        Returns (o, g): o shaped like q, g (bh, nq) or (b, h, nq) float32; with ``save`` also the
        workspace tensor that ``backward(..., saved=...)`` can reuse.  ``out``, ``g`` and ``ws`` (a uint8
        tensor of at least ``workspace_bytes(desc)[0]`` bytes, 256-byte aligned) may be the caller's: a
        call that is given all three allocates nothing and asks the library nothing beforehand."""
        if save:
            flags |= FLAG_SAVE_FOR_BACKWARD
        desc = self.make_desc(q, k, v, mask=mask, inv_tau=inv_tau, a0=a0, a1=a1, a2=a2, p=p, chunk=chunk, flags=flags,
                              norm=norm)
        lead = tuple(q.shape[:-2])
        if out is None:
            out = torch.empty(lead + (desc.nq, desc.d), dtype=q.dtype, device=q.device)
        if g is None:
            g = torch.empty(lead + (desc.nq,), dtype=torch.float32, device=q.device)
        desc.so = _strides(out)
        desc.sg = _gstrides(g)
        if ws is None:
            fwd, _ = self.workspace_bytes(desc)
            ws = self._workspace(fwd, q.device)
        st = self.lib.fastmax_forward(C.byref(desc), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                      g.data_ptr(), ws.data_ptr(), ws.numel(), self._stream(q))
        self.check(st, "fastmax_forward")
        if save:
            return out, g, ws
        return out, g

    def forward_static(self, q, k, v, out, g, *, mask, inv_tau, a0=1.0, a1=1.0, a2=0.5, p=2, chunk=0, flags=0):
        """fastmax_forward_static: the forward on the library's own static scratch buffer.  The caller owns
        ``out`` (shaped like q) and ``g``; nothing is allocated here or in the library."""
        desc = self.make_desc(q, k, v, mask=mask, inv_tau=inv_tau, a0=a0, a1=a1, a2=a2, p=p, chunk=chunk, flags=flags)
        desc.so = _strides(out)
        desc.sg = _gstrides(g)
        st = self.lib.fastmax_forward_static(C.byref(desc), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                             g.data_ptr(), self._stream(q))
        self.check(st, "fastmax_forward_static")
        return out, g

    # -- incremental decoding on a persistent moment state ---------------------------
    def decode_state(self, k, *, inv_tau, p=2, a0=1.0, a1=1.0, a2=0.5):
        """An empty state for tensors shaped like k ((bh, n, d) or (b, h, n, d)): zero-filled float32."""
        desc = self.make_desc(k, k, k, mask=True, inv_tau=inv_tau, a0=a0, a1=a1, a2=a2, p=p)
        return torch.zeros(self.lib.fastmax_decode_state_bytes(C.byref(desc)) // 4, dtype=torch.float32, device=k.device)

    def decode_absorb(self, k, v, state, *, inv_tau, p=2, a0=1.0, a1=1.0, a2=0.5):
        """Adds all tokens of k, v to the state."""
        desc = self.make_desc(k, k, v, mask=True, inv_tau=inv_tau, a0=a0, a1=a1, a2=a2, p=p)
        st = self.lib.fastmax_decode_absorb(C.byref(desc), k.data_ptr(), v.data_ptr(), state.data_ptr(), self._stream(k))
        self.check(st, "fastmax_decode_absorb")

    def decode_step(self, q, k, v, state, *, inv_tau, p=2, a0=1.0, a1=1.0, a2=0.5):
        """One token: q, k, v are (bh, 1, d) or (b, h, 1, d); returns (o, g) for it and updates the state."""
        desc = self.make_desc(q, k, v, mask=True, inv_tau=inv_tau, a0=a0, a1=a1, a2=a2, p=p)
        lead = tuple(q.shape[:-2])
        o = torch.empty(lead + (1, desc.d), dtype=q.dtype, device=q.device)
        g = torch.empty(lead + (1,), dtype=torch.float32, device=q.device)
        desc.so, desc.sg = _strides(o), _gstrides(g)
        scratch = torch.empty(max(self.lib.fastmax_decode_scratch_bytes(C.byref(desc)) // 4, 1), dtype=torch.float32,
                              device=q.device)
        st = self.lib.fastmax_decode_step(C.byref(desc), q.data_ptr(), k.data_ptr(), v.data_ptr(), state.data_ptr(),
                                          o.data_ptr(), g.data_ptr(), scratch.data_ptr(), self._stream(q))
        self.check(st, "fastmax_decode_step")
        return o, g

    def backward(self, q, k, v, o, g, d_o, *, mask, inv_tau, a0=1.0, a1=1.0, a2=0.5, p=2, chunk=0, flags=0,
                 saved: Optional[torch.Tensor] = None, out=None, ws: Optional[torch.Tensor] = None, norm=None):
        """Gradients (dq, dk, dv) of sum(o * d_o); all tensors are (bh, n, d) views.
        ``saved``: the workspace returned by ``forward(..., save=True)`` for the same problem.
        ``out``: caller-owned (dq, dk, dv); ``ws``: caller-owned workspace (see ``forward``)."""
        if saved is not None:
            flags |= FLAG_SAVE_FOR_BACKWARD
        desc = self.make_desc(q, k, v, mask=mask, inv_tau=inv_tau, a0=a0, a1=a1, a2=a2, p=p, chunk=chunk, flags=flags,
                              norm=norm)
        if o.dtype != q.dtype or d_o.dtype != q.dtype or g.dtype != torch.float32:
            raise FastmaxError("fastmax: o and d_o must have q's dtype and g must be float32")
        lead = tuple(q.shape[:-2])
        if out is not None:
            dq, dk, dv = out
        else:
            dq = torch.empty(lead + (desc.nq, desc.d), dtype=q.dtype, device=q.device)
            dk = torch.empty(lead + (desc.nk, desc.d), dtype=q.dtype, device=q.device)
            dv = torch.empty(lead + (desc.nk, desc.d), dtype=q.dtype, device=q.device)
        desc.so, desc.sdo = _strides(o), _strides(d_o)
        desc.sg = _gstrides(g)
        desc.sdq, desc.sdk, desc.sdv = _strides(dq), _strides(dk), _strides(dv)
        if ws is None:
            _, bwd = self.workspace_bytes(desc)
            ws = self._workspace(bwd, q.device)
        bwd = ws.numel()
        if saved is not None:
            st = self.lib.fastmax_backward_saved(C.byref(desc), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                                 g.data_ptr(), d_o.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                                 dv.data_ptr(), saved.data_ptr(), saved.numel(), ws.data_ptr(), bwd,
                                                 self._stream(q))
        else:
            st = self.lib.fastmax_backward(C.byref(desc), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                           g.data_ptr(), d_o.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                           ws.data_ptr(), bwd, self._stream(q))
        self.check(st, "fastmax_backward")
        return dq, dk, dv

    def normalize(self, x, *, centre=0, max_norm=True, scale=1.0, out: Optional[torch.Tensor] = None):
        """x (bh, n, d) view; returns y = scale * (x - centre) / max_n ||.|| (see the header)."""
        nd = NormDesc()
        nd.bh, nd.n, nd.d = _dims(x)
        nd.dtype = _dtype_code(x)
        nd.centre, nd.max_norm, nd.scale = int(centre), int(bool(max_norm)), float(scale)
        if out is None:
            out = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
        nd.sx, nd.sy = _strides(x), _strides(out)
        nbytes = self.lib.fastmax_normalize_stats_bytes(C.byref(nd))
        stats = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=x.device)
        st = self.lib.fastmax_normalize(C.byref(nd), x.data_ptr(), out.data_ptr(), stats.data_ptr(), self._stream(x))
        self.check(st, "fastmax_normalize")
        return out

    def normalize_backward(self, x, dy, *, centre=0, max_norm=True, scale=1.0):
        """Gradient of normalize() with respect to x; x and dy are (bh, n, d) views."""
        nd = NormDesc()
        nd.bh, nd.n, nd.d = _dims(x)
        nd.dtype = _dtype_code(x)
        nd.centre, nd.max_norm, nd.scale = int(centre), int(bool(max_norm)), float(scale)
        x = x.contiguous()                 # dx is written with x's strides
        dx = torch.empty_like(x)
        nd.sx, nd.sy = _strides(x), _strides(dy)
        nbytes = self.lib.fastmax_normalize_backward_stats_bytes(C.byref(nd))
        stats = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=x.device)
        st = self.lib.fastmax_normalize_backward(C.byref(nd), x.data_ptr(), dy.data_ptr(), dx.data_ptr(), stats.data_ptr(),
                                                 self._stream(x))
        self.check(st, "fastmax_normalize_backward")
        return dx

    def _pointwise_desc(self, x, out):
        nd = NormDesc()
        nd.bh, nd.n, nd.d = _dims(x)
        nd.dtype = _dtype_code(x)
        nd.sx, nd.sy = _strides(x), _strides(out)
        return nd

    def key_rpe(self, k, rpe, temperature: float, out: Optional[torch.Tensor] = None):
        """k (bh, n, d) view, rpe (2n-1, d): k + temperature * rpe[(l + n) % (2n - 1)], the keys that make the
        operator see k / temperature + rpe (the addition the reference leaves commented out)."""
        bh, n, d = _dims(k)
        if tuple(rpe.shape) != (2 * n - 1, d):
            raise ValueError(f"rpe must be ({2 * n - 1}, {d}), got {tuple(rpe.shape)}")
        table = rpe.detach().to(device=k.device, dtype=torch.float32).contiguous()
        if out is None:
            out = torch.empty(tuple(k.shape), dtype=k.dtype, device=k.device)
        nd = self._pointwise_desc(k, out)
        st = self.lib.fastmax_key_rpe(C.byref(nd), k.data_ptr(), table.data_ptr(), out.data_ptr(), float(temperature),
                                      self._stream(k))
        self.check(st, "fastmax_key_rpe")
        return out

    def output_noise(self, o, noise, scale: float, out: Optional[torch.Tensor] = None):
        """o * (1 + scale * noise); o and noise (bh, n, d) views of one type and layout."""
        if noise.dtype != o.dtype or tuple(noise.shape) != tuple(o.shape) or noise.stride() != o.stride():
            raise ValueError("noise must have o's type, shape and strides")
        if out is None:
            out = torch.empty(tuple(o.shape), dtype=o.dtype, device=o.device)
        nd = self._pointwise_desc(o, out)
        st = self.lib.fastmax_output_noise(C.byref(nd), o.data_ptr(), noise.data_ptr(), out.data_ptr(), float(scale),
                                           self._stream(o))
        self.check(st, "fastmax_output_noise")
        return out

    KERNEL_NAMES = ("transpose", "prep_bwd", "build", "fwd", "dq", "dk", "normalize", "dv", "dkv")

    # -- bench aids (only in the library built with -DFM_BENCH_AIDS) --------------------
    def profile_begin(self) -> None:
        self.lib.fastmax_profile_begin()

    def profile_end(self, capacity: int = 4096):
        """[(kernel name, milliseconds)] for every launch since profile_begin()."""
        ids = (C.c_int * capacity)()
        ms = (C.c_float * capacity)()
        n = min(self.lib.fastmax_profile_end(ids, ms, capacity), capacity)
        return [(self.KERNEL_NAMES[ids[i]], float(ms[i])) for i in range(n)]

    def probe_lds_transpose(self, device):
        """(64 lanes, 4) values the transposing LDS read returns for the header's test pattern."""
        out = torch.zeros(256, dtype=torch.float32, device=device)
        self.check(self.lib.fastmax_probe_lds_transpose(out.data_ptr(), 0), "fastmax_probe_lds_transpose")
        return out.view(64, 4)

    def probe_mfma(self, device):
        a = torch.zeros(1024, dtype=torch.float32, device=device)
        b = torch.zeros(1024, dtype=torch.float32, device=device)
        self.check(self.lib.fastmax_probe_mfma(a.data_ptr(), b.data_ptr(), 0), "fastmax_probe_mfma")
        return a.view(64, 16), b.view(64, 16)

    def mfma_rate(self, device, workgroups: int = 2048, iters: int = 4000) -> float:
        """TFLOP/s of a register-only loop of 32x32x16 _Float16 matrix products on `device`
        (event-timed on torch's current stream after one short warm-up launch)."""
        out = torch.empty(workgroups * 256, dtype=torch.float32, device=device)
        stream = torch.cuda.current_stream(out.device).cuda_stream
        self.check(self.lib.fastmax_probe_mfma_rate(workgroups, 10, out.data_ptr(), stream), "fastmax_probe_mfma_rate")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        self.check(self.lib.fastmax_probe_mfma_rate(workgroups, iters, out.data_ptr(), stream), "fastmax_probe_mfma_rate")
        e1.record()
        e1.synchronize()
        return workgroups * 4 * iters * 8 * 32768.0 / (e0.elapsed_time(e1) * 1e-3) / 1e12

    def mix_rate(self, device, own_tiles: int = 1, iters: int = 4000) -> float:
        """TFLOP/s of the matrix products of a loop with the dense kernels' instruction mix (operands read
        out of LDS, packed-half vector work beside them; see fastmax_probe_mix_rate), every CU filled the
        way the dK + dV pass fills it."""
        workgroups = 512 if own_tiles == 1 else 256
        out = torch.empty(workgroups * 256, dtype=torch.float32, device=device)
        stream = torch.cuda.current_stream(out.device).cuda_stream
        self.check(self.lib.fastmax_probe_mix_rate(workgroups, 10, own_tiles, out.data_ptr(), stream), "fastmax_probe_mix_rate")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        self.check(self.lib.fastmax_probe_mix_rate(workgroups, iters, own_tiles, out.data_ptr(), stream), "fastmax_probe_mix_rate")
        e1.record()
        e1.synchronize()
        return workgroups * 4 * iters * 16 * own_tiles * 32768.0 / (e0.elapsed_time(e1) * 1e-3) / 1e12


_lock = threading.Lock()
_default: Optional[FastmaxLib] = None


def get_lib() -> FastmaxLib:
    """The process-wide library handle (loaded on first use)."""
    global _default
    with _lock:
        if _default is None:
            _default = FastmaxLib()
        return _default


_bench: Optional[FastmaxLib] = None


def get_bench_lib() -> FastmaxLib:
    """The bench build of the same sources (per-kernel event timing, matrix-rate yardsticks)."""
    global _bench
    with _lock:
        if _bench is None:
            _bench = FastmaxLib(bench=True)
        return _bench
