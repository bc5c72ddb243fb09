"""CPU run of the kernel sources through the host simulator (tests/hostsim/hostsim.h).

The very same kernel templates the GPU runs are compiled as plain C++ with
-DFM_HOSTSIM (work-items are OS threads, MFMA tiles are emulated with the lane
layout the GPU probe test pins) and driven through the same C ABI.  This checks
indexing, lane layouts, masks and ragged sizes without a GPU and, with
FASTMAX_HOSTSIM_ASAN=1 (minutes of compile and run time, so not by default), under
AddressSanitizer through a driver of its own (tests/hostsim/asan_driver.cpp).  It is a test build
only: the package never loads it.  Sizes are tiny because every work-item is a thread.
"""
import os
import shutil
import subprocess

import pytest
import torch

from reproducing_fastmax_results_amd import _capi
from tests.parity import (TOL, check_batch_head_strides, check_decode, check_norm_fold, check_forward, check_forward_backward, make_inputs, oracle_all,
                          rel_err)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLANG = shutil.which("clang++", path="/opt/rocm/llvm/bin:" + os.environ.get("PATH", ""))

pytestmark = pytest.mark.skipif(CLANG is None, reason="no clang++ for the host simulator build")


@pytest.fixture(scope="module")
def sim(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("hostsim") / "libfastmax_hostsim.so")
    cmd = [CLANG, "-x", "c++", "-std=c++17", "-O2", "-DFM_HOSTSIM", "-Wno-psabi", "-fPIC", "-shared", "-pthread",
           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "tests", "hostsim"),
           "-I", os.path.join(ROOT, "reproducing_fastmax_results_amd", "csrc"),
           os.path.join(ROOT, "reproducing_fastmax_results_amd", "csrc", "fastmax_api.hip"), "-o", out]
    subprocess.run(cmd, check=True, capture_output=True)
    return _capi.FastmaxLib(out)


def test_probe_matches_assumed_layout(sim):
    a16, a32 = sim.probe_mfma("cpu")
    lane = torch.arange(64).view(64, 1)
    e = torch.arange(16).view(1, 16)
    want = ((8 * (e // 4) + 4 * (lane // 32) + e % 4 + 1) * 100 + lane % 32 + 1).float()
    assert torch.equal(a16, want) and torch.equal(a32, want)


def test_lds_transpose_read_matches_assumed_layout(sim):
    got = sim.probe_lds_transpose("cpu")
    lane = torch.arange(64).view(64, 1)
    t = torch.arange(4).view(1, 4)
    assert torch.equal(got, (64 * (4 * t + (lane % 16) // 4) + 4 * (lane // 16) + lane % 4).float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_forward_backward(sim, dtype):
    check_forward_backward(sim, 1, 70, 32, dtype, "cpu", mask=True, p=2, flags=_capi.FLAG_FORCE_DENSE, seed=1)
    check_forward_backward(sim, 1, 33, 32, dtype, "cpu", mask=False, p=1, nk=45, seed=2)


def test_moment_path_forward_backward_bf16(sim):
    # two segments of 256: prefix state for the second, suffix state for the first
    check_forward_backward(sim, 1, 300, 32, torch.bfloat16, "cpu", mask=True, p=2, chunk=256, seed=3)
    check_forward_backward(sim, 1, 300, 32, torch.bfloat16, "cpu", mask=True, p=2, chunk=256, seed=3, saved=True)
    check_forward_backward(sim, 1, 40, 32, torch.bfloat16, "cpu", mask=False, p=2, nk=260,
                           flags=_capi.FLAG_FORCE_MOMENTS, seed=4)


def test_order1_segments_summed_apart_then_scanned(sim):
    # order 1 with three segments: each segment's sums come from its own workgroups and
    # an elementwise scan over the segments makes the prefix and suffix states
    check_forward_backward(sim, 1, 600, 32, torch.bfloat16, "cpu", mask=True, p=1, chunk=256, seed=9)
    check_forward_backward(sim, 1, 600, 32, torch.float32, "cpu", mask=True, p=1, chunk=256, seed=10, saved=True)
    check_forward_backward(sim, 1, 40, 32, torch.bfloat16, "cpu", mask=False, p=1, nk=300,
                           flags=_capi.FLAG_FORCE_MOMENTS, seed=11)


def test_batch_and_head_strides(sim):
    # (b, n, h*d) projections viewed as (b, h, n, d): FastmaxStrides with heads > 1
    check_batch_head_strides(sim, 2, 2, 70, 32, torch.bfloat16, "cpu", mask=True, p=2, seed=7)
    check_batch_head_strides(sim, 2, 2, 40, 32, torch.float32, "cpu", mask=False, p=1, seed=8)
    # one head per batch: stride(1) of the transposed (b, n, 1, d) view is d, the slices lie n*d apart
    check_batch_head_strides(sim, 3, 1, 40, 32, torch.bfloat16, "cpu", mask=True, p=2, seed=9)
    check_batch_head_strides(sim, 3, 1, 33, 32, torch.float32, "cpu", mask=False, p=2, seed=10)


def test_moment_path_forward_fp32_d64(sim):
    check_forward(sim, 1, 290, 64, torch.float32, "cpu", mask=True, p=2, chunk=256, seed=5)


def test_normalize(sim):
    from oracle import fastmax_oracle as O
    x = torch.randn(2, 70, 32, generator=torch.Generator().manual_seed(6))
    for centre, ref in ((0, O.normalize_lim(x.double(), 1.5)),
                        (1, 1.5 * O.normalize_feature_mean(x.double(), x.double())[0]),
                        (2, 1.5 * O.normalize_token_mean(x.double(), x.double())[0])):
        y = sim.normalize(x, centre=centre, max_norm=True, scale=1.5)
        assert O.rel_l2(y, ref) < 1e-6
    y = sim.normalize(x, centre=0, max_norm=False, scale=0.25)
    assert torch.allclose(y, 0.25 * x)
    # several workgroups per batch*head: their partial maxima and column sums are joined by the last kernel
    x = torch.randn(3, 600, 64, generator=torch.Generator().manual_seed(7))
    x[1, 555] *= 3.0
    for centre, ref in ((0, O.normalize_lim(x.double(), 0.5)), (2, 0.5 * O.normalize_token_mean(x.double(), x.double())[0])):
        assert O.rel_l2(sim.normalize(x, centre=centre, max_norm=True, scale=0.5), ref) < 1e-6
    assert O.rel_l2(sim.normalize(x, centre=2, max_norm=False, scale=2.0), 2.0 * (x - x.mean(1, keepdim=True)).double()) < 1e-6


def test_dormant_steps(sim):
    """Key RPE and output noise (the reference's switched-off steps) on ragged sizes and both types."""
    from oracle import fastmax_oracle as O
    for shape, dtype in (((2, 70, 32), torch.float32), ((1, 2, 129, 64), torch.bfloat16), ((1, 1, 64), torch.float32)):
        n, d = shape[-2], shape[-1]
        gen = torch.Generator().manual_seed(61)
        k = torch.randn(*shape, generator=gen).to(dtype)
        rpe = torch.randn(2 * n - 1, d, generator=gen)
        noise = torch.randn(*shape, generator=gen).to(dtype)
        tol = 1e-6 if dtype == torch.float32 else 4e-3
        assert O.rel_l2(sim.key_rpe(k, rpe, 2.5), O.apply_rpe_and_temp(k.double(), rpe, 2.5) * 2.5) < tol
        assert O.rel_l2(sim.output_noise(k, noise, -0.4), O.apply_dropout(k, noise, -0.4)) < tol
        assert torch.equal(sim.output_noise(k, noise, 0.0), k)


def test_normalize_backward(sim):
    from oracle import fastmax_oracle as O
    g = torch.Generator().manual_seed(12)
    x, dy = torch.randn(2, 150, 32, generator=g), torch.randn(2, 150, 32, generator=g)
    for centre, fn in ((0, lambda t: O.normalize_lim(t, 1.5)),
                       (1, lambda t: 1.5 * O.normalize_feature_mean(t, t)[0]),
                       (2, lambda t: 1.5 * O.normalize_token_mean(t, t)[0])):
        xd = x.double().requires_grad_(True)
        fn(xd).backward(dy.double())
        dx = sim.normalize_backward(x, dy, centre=centre, max_norm=True, scale=1.5)
        assert O.rel_l2(dx, xd.grad) < 1e-5
    x, dy = torch.randn(2, 600, 64, generator=g), torch.randn(2, 600, 64, generator=g)
    xd = x.double().requires_grad_(True)
    (1.5 * O.normalize_token_mean(xd, xd)[0]).backward(dy.double())
    assert O.rel_l2(sim.normalize_backward(x, dy, centre=2, max_norm=True, scale=1.5), xd.grad) < 1e-5


def test_order2_walk_per_value_column(sim):
    """k_walk_sym (D = 64, _Float16): prefix walk for the forward, suffix walk with the weights c for the backward,
    dQ reading the forward's state transposed; with and without the forward's kept workspace, and the one global
    state of unmasked attention."""
    check_forward_backward(sim, 1, 300, 64, torch.bfloat16, "cpu", mask=True, p=2, chunk=256, seed=21)
    check_forward_backward(sim, 1, 512, 64, torch.bfloat16, "cpu", mask=True, p=2, chunk=256, seed=22, saved=True)
    check_forward_backward(sim, 1, 130, 64, torch.bfloat16, "cpu", mask=False, p=2, nk=300, seed=23, flags=_capi.FLAG_FORCE_MOMENTS)


def test_causal_with_more_keys_than_queries(sim):
    # query i sees keys 0 .. nk - nq + i (fastmax_cuda_forward.cu:161-172): head + square tail, merged
    check_forward_backward(sim, 1, 40, 32, torch.float32, "cpu", mask=True, p=2, nk=75, seed=13)
    check_forward_backward(sim, 2, 33, 32, torch.bfloat16, "cpu", mask=True, p=1, nk=34, seed=14)



def test_segment_length_sentinels(sim):
    # a segment length at or beyond the sequence means "one segment", whatever its size; beyond 2^30 it is rejected
    import ctypes as C
    q, k, v, go = make_inputs(1, 300, 300, 32, torch.float32, "cpu", seed=15)
    kw = dict(mask=True, inv_tau=0.1, p=2)
    o0, g0 = sim.forward(q, k, v, chunk=0, **kw)
    for chunk in (300, 301, 1 << 20, 1 << 30):
        o1, g1 = sim.forward(q, k, v, chunk=chunk, **kw)
        assert torch.equal(o0, o1) and torch.equal(g0, g1)
    for chunk in ((1 << 30) + 1, 2 ** 31 - 1):
        d = sim.make_desc(q, k, v, mask=True, inv_tau=0.1, a0=1.0, a1=1.0, a2=0.5, p=2, chunk=chunk)
        assert sim.lib.fastmax_workspace_bytes(C.byref(d), None, None) == 2
    d = sim.make_desc(q, k, v, mask=True, inv_tau=0.1, a0=1.0, a1=1.0, a2=0.5, p=2)
    d.nq = d.nk = (1 << 30) + 1
    assert sim.lib.fastmax_workspace_bytes(C.byref(d), None, None) == 2


def _domain_case(sim, scale, flags, a=(1.0, 1.0, 0.5)):
    bh, n, d = 1, 70, 32
    q, k, v, go = make_inputs(bh, n, n, d, torch.bfloat16, "cpu", seed=16, scale=scale)
    kw = dict(mask=True, inv_tau=1.0, a0=a[0], a1=a[1], a2=a[2], p=2, flags=flags)
    o, g = sim.forward(q, k, v, **kw)
    grads = sim.backward(q, k, v, o, g, go, **kw)
    ref = oracle_all(q, k, v, go, mask=True, tau=1.0, p=2, a=a)
    smax = float((q.double() @ k.double().transpose(1, 2)).abs().max())
    return smax, [(x, r) for x, r in zip((o, g) + tuple(grads), ref)]


def test_bf16_range_is_loud_not_wrong(sim):
    """bf16 tensors are computed in _Float16.  Inside the documented range (|s| <= 250) the results meet
    the bf16 bar; beyond it every result is either still within the bar or not finite - never a finite
    wrong number; and with FASTMAX_FLAG_F32_COMPUTE the same inputs meet the bar."""
    smax, pairs = _domain_case(sim, 2.2, 0)                         # |s| up to about 200
    assert 100.0 < smax <= 250.0
    for x, r in pairs:
        assert bool(torch.isfinite(x).all()) and rel_err(x, r) < TOL[torch.bfloat16]
    for scale in (8.0, 30.0, 300.0):                               # |s| ~ 2e3, 3e4, 3e6
        smax, pairs = _domain_case(sim, scale, 0)
        assert smax > 362.0
        for x, r in pairs:
            assert (not bool(torch.isfinite(x).all())) or rel_err(x, r) < TOL[torch.bfloat16]
        _, pairs = _domain_case(sim, scale, _capi.FLAG_F32_COMPUTE)
        for x, r in pairs:
            assert bool(torch.isfinite(x).all()) and rel_err(x, r) < TOL[torch.bfloat16]
    # a0 = 0: denominators no longer grow with the token index (g_0 = s + s^2 / 2 can be tiny)
    _, pairs = _domain_case(sim, 1.0, _capi.FLAG_F32_COMPUTE, a=(0.0, 1.0, 0.5))
    for x, r in pairs:
        assert bool(torch.isfinite(x).all()) and rel_err(x, r) < TOL[torch.bfloat16]
    _, pairs = _domain_case(sim, 1.0, 0, a=(0.0, 1.0, 0.5))            # a0 <= 0: fp32 arithmetic without being asked
    for x, r in pairs:
        assert bool(torch.isfinite(x).all()) and rel_err(x, r) < TOL[torch.bfloat16]


def test_normalize_zero_slice(sim):
    # an all-zero (b, h) slice (padding) comes out as zeros with zero gradient, not 0 / 0
    g = torch.Generator().manual_seed(17)
    x, dy = torch.randn(3, 70, 32, generator=g), torch.randn(3, 70, 32, generator=g)
    x[1] = 0.0
    y = sim.normalize(x, centre=0, max_norm=True, scale=1.5)
    assert bool(torch.isfinite(y).all()) and float(y[1].abs().max()) == 0.0
    dx = sim.normalize_backward(x, dy, centre=0, max_norm=True, scale=1.5)
    assert bool(torch.isfinite(dx).all()) and float(dx[1].abs().max()) == 0.0


def test_upstream_gradient_of_any_size(sim):
    # gradients are linear in dO, whose size is the caller's (a mean-reduced loss: 1e-6 and less): the bf16
    # path scales dO / g per batch*head to the _Float16 range and back (k_grad_scale)
    for go_scale in (1e-7, 3e4):
        check_forward_backward(sim, 2, 70, 32, torch.bfloat16, "cpu", mask=True, p=2, flags=_capi.FLAG_FORCE_DENSE,
                               seed=20, go_scale=go_scale)
        check_forward_backward(sim, 1, 300, 32, torch.bfloat16, "cpu", mask=True, p=2, chunk=256, seed=21,
                               go_scale=go_scale, saved=True)
    check_forward_backward(sim, 1, 300, 32, torch.bfloat16, "cpu", mask=True, p=1, chunk=256, seed=22, go_scale=1e-7)


def test_normalisation_folded_into_the_loads(sim):
    # q and k normalised as they are loaded; gradients through the normalisation (one row gets the rank-one term)
    check_norm_fold(sim, 2, 70, 32, torch.float32, "cpu", mask=True, p=2, seed=23)
    check_norm_fold(sim, 2, 70, 32, torch.bfloat16, "cpu", mask=True, p=2, seed=24)
    check_norm_fold(sim, 1, 300, 32, torch.bfloat16, "cpu", mask=True, p=2, chunk=256, seed=25)      # through states
    check_norm_fold(sim, 1, 300, 32, torch.float32, "cpu", mask=True, p=1, chunk=256, seed=26, saved=False)
    check_norm_fold(sim, 2, 40, 32, torch.float32, "cpu", mask=False, p=2, nk=75, seed=27, saved=False)
    # the reference extension's gradients: with respect to the normalised tensors
    check_norm_fold(sim, 2, 70, 32, torch.float32, "cpu", mask=True, p=2, seed=28, jacobian=False)


def test_incremental_decoding_on_the_moment_state(sim):
    # a prompt absorbed into the state, then one step per token; and decoding from the empty state
    check_decode(sim, 2, 40, 33, 32, torch.float32, "cpu", p=2, seed=30)
    check_decode(sim, 2, 12, 0, 32, torch.bfloat16, "cpu", p=2, seed=31, tau_mult=1.0)
    check_decode(sim, 2, 30, 20, 32, torch.float32, "cpu", p=1, seed=32, four_d=True)


def test_prompt_absorbed_with_matrix_instructions(sim):
    # bf16, D = 64, order 2, 64 tokens or more: k_decode_absorb_mma (two tiles here, the second ragged), then steps
    check_decode(sim, 1, 134, 130, 64, torch.bfloat16, "cpu", p=2, seed=33)
    # the same sums as token by token (k_decode), also added to a state that is not empty
    import math
    q, k, v, _ = make_inputs(1, 100, 100, 64, torch.bfloat16, "cpu", 5)
    kw = dict(inv_tau=1.0 / (8 * math.sqrt(64)), p=2, a0=1.0, a1=1.0, a2=0.5)
    s1, s2 = sim.decode_state(k, **kw), sim.decode_state(k, **kw)
    sim.decode_absorb(k[:, :30], v[:, :30], s1, **kw)          # k_decode
    sim.decode_absorb(k[:, 30:], v[:, 30:], s1, **kw)          # 70 tokens: matrix instructions, into a state that is not empty
    sim.decode_absorb(k[:, :50], v[:, :50], s2, **kw)
    sim.decode_absorb(k[:, 50:], v[:, 50:], s2, **kw)
    assert float((s1 - s2).norm() / s2.norm()) < 1e-5
    live = s2.abs() > 1e-3 * s2.abs().max()
    assert float(((s1 - s2).abs() / s2.abs().clamp_min(1e-30))[live].max()) < 5e-3      # operands rounded to _Float16


def test_bf16_value_range_on_the_cpu(sim):
    # the range of v the header states for bf16 tensors: 1e2 within the bar, beyond it within the bar or not finite
    import math
    bh, n, d = 1, 70, 32
    tau = 8.0 * math.sqrt(d)
    for vs, inside in ((1e2, True), (1e3, False), (1e4, False)):
        gen = torch.Generator().manual_seed(3)
        q, k = (torch.randn(bh, n, d, generator=gen).bfloat16() for _ in range(2))
        v = (vs * torch.randn(bh, n, d, generator=gen)).bfloat16()
        go = torch.randn(bh, n, d, generator=gen).bfloat16()
        kw = dict(mask=True, inv_tau=1.0 / tau, p=2)
        o, g, ws = sim.forward(q, k, v, save=True, **kw)
        grads = sim.backward(q, k, v, o, g, go, saved=ws, **kw)
        ref = oracle_all(q, k, v, go, mask=True, tau=tau, p=2)
        for x, r in zip((o, g) + tuple(grads), ref):
            ok = rel_err(x, r) < TOL[torch.bfloat16]
            assert ok if inside else (ok or not bool(torch.isfinite(x).all())), f"v x {vs:g}"


def test_heads_of_128(sim):
    # bf16 tensors, D = 128: the _Float16 token kernels on dense tiles, four accumulator tiles per feature axis
    check_forward_backward(sim, 1, 70, 128, torch.bfloat16, "cpu", mask=True, p=2, seed=50, saved=True)
    check_forward_backward(sim, 1, 40, 128, torch.bfloat16, "cpu", mask=False, p=1, nk=75, seed=51)


def test_order1_segment_backward_in_one_pass(sim):
    # beyond 1024 tokens order 1 on _Float16 runs in 128-token segments and k_o1_bwd makes dq, dk, dv of a segment
    # in one workgroup (9 segments here, the last one ragged); also with the folded normalisation's Jacobian
    check_forward_backward(sim, 1, 1100, 32, torch.bfloat16, "cpu", mask=True, p=1, seed=40, saved=True)
    check_norm_fold(sim, 1, 1100, 32, torch.bfloat16, "cpu", mask=True, p=1, seed=41)


@pytest.mark.skipif(os.environ.get("FASTMAX_HOSTSIM_ASAN") != "1", reason="set FASTMAX_HOSTSIM_ASAN=1 (several minutes)")
def test_kernel_sources_under_address_sanitizer(tmp_path):
    # the state walk with two tile buffers, order 1 in runs of segments, the dense kernels, fp32: forward and backward
    exe = str(tmp_path / "asan_driver")
    cmd = [CLANG, "-x", "c++", "-std=c++17", "-O1", "-g", "-DFM_HOSTSIM", "-Wno-psabi", "-pthread", "-fsanitize=address",
           "-fno-omit-frame-pointer", "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "tests", "hostsim"),
           "-I", os.path.join(ROOT, "reproducing_fastmax_results_amd", "csrc"),
           os.path.join(ROOT, "reproducing_fastmax_results_amd", "csrc", "fastmax_api.hip"),
           os.path.join(ROOT, "tests", "hostsim", "asan_driver.cpp"), "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True)
    run = subprocess.run([exe], capture_output=True, text=True, env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0"))
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-4000:]
    assert "AddressSanitizer" not in run.stderr
