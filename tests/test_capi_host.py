"""CPU-side tests of the C ABI: the library loads, exports every symbol the header declares,
and rejects bad arguments with the documented status codes (no kernel is launched)."""
import ctypes as C
import os
import re

import pytest

from reproducing_fastmax_results_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "reproducing_fastmax_results_amd", _capi.LIB_NAME)

pytestmark = pytest.mark.skipif(not os.path.exists(LIB), reason="libfastmax_hip.so not built (run __graft_entry__.build())")


@pytest.fixture(scope="module")
def lib():
    return _capi.FastmaxLib(LIB)


def declared_functions():
    text = open(os.path.join(ROOT, "include", "fastmax_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fastmax_[a-z_0-9]+)\s*\(", text)))


def test_exports_match_header(lib):
    names = declared_functions()
    assert set(names) == set(_capi.EXPORTS)
    for n in names:
        assert getattr(lib.lib, n) is not None


def test_bench_build_exports_the_aids_on_top(lib):
    """libfastmax_hip_bench.so: everything the product exports plus the bench aids; the product has none of them."""
    path = os.path.join(ROOT, "reproducing_fastmax_results_amd", _capi.BENCH_LIB_NAME)
    if not os.path.exists(path):
        pytest.skip("bench build of the library not built")
    bench = _capi.FastmaxLib(path, bench=True)
    for n in _capi.EXPORTS + _capi.BENCH_EXPORTS:
        assert getattr(bench.lib, n) is not None
    for n in _capi.BENCH_EXPORTS:
        assert not hasattr(lib.lib, n)
    one = C.c_void_p(256)
    assert bench.lib.fastmax_probe_mfma_rate(1, 1, None, None) == 1
    assert bench.lib.fastmax_probe_mfma_rate(0, 1, one, None) == 2
    assert bench.lib.fastmax_probe_mfma_rate(1, (1 << 20) + 1, one, None) == 2


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(ImportError, match="no CPU fallback"):
        _capi.FastmaxLib(str(tmp_path / "libfastmax_hip.so"))


def base_desc(**kw):
    d = _capi.Desc()
    d.bh, d.nq, d.nk, d.d = 4, 128, 128, 64
    d.dtype, d.mask, d.p = _capi.BF16, 1, 2
    d.a0, d.a1, d.a2, d.inv_tau = 1.0, 1.0, 0.5, 0.125
    for name in ("sq", "sk", "sv", "so", "sdo", "sdq", "sdk", "sdv"):
        setattr(d, name, _capi.Strides(128 * 64, 64))
    d.sg = _capi.Strides(128, 1)
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def ws(lib, d):
    f, b = C.c_size_t(0), C.c_size_t(0)
    st = lib.lib.fastmax_workspace_bytes(C.byref(d), C.byref(f), C.byref(b))
    return st, f.value, b.value


def test_workspace_sizes_and_status_codes(lib):
    st, f, b = ws(lib, base_desc())
    assert st == 0 and f >= 256 and b >= f
    assert ws(lib, base_desc(d=48))[0] == 3          # unsupported head size
    # heads of 128: bf16 tensors on the _Float16 kernels, dense tiles only
    st3, f3, b3 = ws(lib, base_desc(d=128))
    assert st3 == 0 and f3 >= 2 * 4 * 256 * 128 * 2                      # the converted k and v
    assert ws(lib, base_desc(d=128, dtype=_capi.F32))[0] == 3
    assert ws(lib, base_desc(d=128, flags=_capi.FLAG_F32_COMPUTE))[0] == 3
    assert ws(lib, base_desc(d=128, flags=_capi.FLAG_FORCE_MOMENTS, mask=0))[0] == 3
    assert ws(lib, base_desc(d=128, a0=0.0))[0] == 3                     # would need the fp32 kernels
    assert ws(lib, base_desc(d=128, nk=256))[0] == 3                     # causal with more keys than queries
    assert ws(lib, base_desc(d=128, nk=256, mask=0))[0] == 0
    long128 = ws(lib, base_desc(d=128, nq=16384, nk=16384))
    assert long128[0] == 0 and long128[2] < 8 * 4 * 16384 * 128 * 2     # copies of the tensors, no states
    assert ws(lib, base_desc(d=256))[0] == 3
    assert ws(lib, base_desc(p=3))[0] == 3           # unsupported order
    assert ws(lib, base_desc(nq=256))[0] == 3        # masked needs nq <= nk
    st2, f2, b2 = ws(lib, base_desc(nk=256))         # masked, more keys than queries: two parts and a merge
    assert st2 == 0 and f2 > f and b2 > b
    assert ws(lib, base_desc(nk=256, mask=0))[0] == 0
    assert ws(lib, base_desc(dtype=7))[0] == 6
    assert ws(lib, base_desc(bh=0))[0] == 2
    assert lib.lib.fastmax_workspace_bytes(None, None, None) == 1
    # long sequences use the moment scan: scratch grows with the number of segments
    small = ws(lib, base_desc(nq=1024, nk=1024))[1]
    large = ws(lib, base_desc(nq=8192, nk=8192))[1]
    assert large > 8 * small / 2
    for code in range(0, 8):
        assert isinstance(lib.status_string(code), str) and lib.status_string(code)


def test_forward_backward_reject_bad_arguments_before_launching(lib):
    d = base_desc()
    one = C.c_void_p(256)     # never dereferenced: validation fails first
    assert lib.lib.fastmax_forward(C.byref(d), None, one, one, one, one, one, 1 << 30, None) == 1
    assert lib.lib.fastmax_forward(C.byref(d), one, one, one, one, one, None, 0, None) == 4      # no workspace
    assert lib.lib.fastmax_forward(C.byref(d), one, one, one, one, one, C.c_void_p(264), 1 << 30, None) == 4  # misaligned
    assert lib.lib.fastmax_forward(C.byref(d), one, one, one, one, one, one, 16, None) == 4     # too small
    bad = base_desc()
    bad.sq = _capi.Strides(128 * 64, 8)               # token stride smaller than the head size
    assert lib.lib.fastmax_forward(C.byref(bad), one, one, one, one, one, one, 1 << 30, None) == 2
    args = [one] * 9
    assert lib.lib.fastmax_backward(C.byref(d), *args, None, 0, None) == 4
    assert lib.lib.fastmax_backward(C.byref(d), None, *args[1:], one, 1 << 30, None) == 1
    # backward on a saved forward workspace: the workspace, its size and the flag are checked
    big = 1 << 30
    assert lib.lib.fastmax_backward_saved(C.byref(d), *args, None, big, one, big, None) == 1          # no forward workspace
    assert lib.lib.fastmax_backward_saved(C.byref(d), *args, one, big, one, big, None) == 2           # flag not set
    ds = base_desc()
    ds.flags = _capi.FLAG_SAVE_FOR_BACKWARD
    assert lib.lib.fastmax_backward_saved(C.byref(ds), *args, one, 16, one, big, None) == 4           # too small
    assert lib.lib.fastmax_backward_saved(C.byref(ds), *args, C.c_void_p(264), big, one, big, None) == 4  # misaligned
    # batch and head strides: heads must divide bh, both strides must be positive
    two = base_desc(bh=8)
    two.sq = _capi.Strides(64, 8 * 64, 128 * 8 * 64, 3)
    assert lib.lib.fastmax_forward(C.byref(two), one, one, one, one, one, one, big, None) == 2
    two.sq = _capi.Strides(64, 8 * 64, 0, 4)
    assert lib.lib.fastmax_forward(C.byref(two), one, one, one, one, one, one, big, None) == 2
    nd = _capi.NormDesc()
    nd.bh, nd.n, nd.d, nd.dtype, nd.centre, nd.max_norm, nd.scale = 2, 10, 40, 0, 0, 1, 1.0
    assert lib.lib.fastmax_normalize(C.byref(nd), one, one, one, None) == 3
    nd.d, nd.centre = 64, 5
    assert lib.lib.fastmax_normalize(C.byref(nd), one, one, one, None) == 3
    nd.centre = 0
    nd.sx = nd.sy = _capi.Strides(640, 64)
    assert lib.lib.fastmax_normalize(C.byref(nd), one, one, None, None) == 4   # max_norm needs stats scratch
    assert lib.lib.fastmax_probe_mfma(None, None, None) == 1
    assert lib.lib.fastmax_probe_lds_transpose(None, None) == 1
    assert lib.lib.fastmax_version() >= 200


def test_static_scratch_entry_rejects_before_touching_the_device(lib):
    # fastmax_forward_static: argument and size checks come before the first HIP call
    one = C.c_void_p(256)
    assert lib.lib.fastmax_forward_static(None, one, one, one, one, one, None) == 1
    assert lib.lib.fastmax_forward_static(C.byref(base_desc(d=48)), one, one, one, one, one, None) == 3
    big = base_desc(bh=16, nq=65536, nk=65536)
    for name in ("sq", "sk", "sv", "so"):
        setattr(big, name, _capi.Strides(65536 * 64, 64))
    big.sg = _capi.Strides(65536, 1)
    st, f, _ = ws(lib, big)
    assert st == 0 and f > _capi.STATIC_SCRATCH_BYTES
    assert lib.lib.fastmax_forward_static(C.byref(big), one, one, one, one, one, None) == 7
    assert "static buffer" in lib.status_string(7)
    # the headline forward (B*H = 32, N = 4096, D = 64, bf16) fits
    c2 = base_desc(bh=32, nq=4096, nk=4096)
    assert ws(lib, c2)[1] <= _capi.STATIC_SCRATCH_BYTES


def test_segment_length_and_size_limits(lib):
    # segment lengths beyond 2^30 and token counts beyond 2^30 are refused (32-bit padding arithmetic)
    assert ws(lib, base_desc(chunk=2 ** 31 - 1))[0] == 2
    assert ws(lib, base_desc(chunk=1 << 30))[0] == 0
    assert ws(lib, base_desc(nq=(1 << 30) + 1, nk=(1 << 30) + 1))[0] == 2
    assert ws(lib, base_desc(chunk=1 << 20))[1] == ws(lib, base_desc())[1]      # "no chunking" sentinel: one segment


def test_normalize_backward_arguments(lib):
    nd = _capi.NormDesc()
    nd.bh, nd.n, nd.d, nd.dtype, nd.centre, nd.max_norm, nd.scale = 4, 130, 64, _capi.F32, 2, 1, 1.0
    nd.sx = nd.sy = _capi.Strides(130 * 64, 64)
    # per batch*head: 4 header floats, the token means of x and dy, one partial sum per 64 tokens (even count),
    # one 8-byte key per 128 tokens, and with the token-mean centring the column sums of x and dy per 256 tokens
    assert lib.lib.fastmax_normalize_backward_stats_bytes(C.byref(nd)) == 4 * 4 * (4 + 2 * 64 + 4 + 2 * 2 + 2 * 64)
    nd.centre = 0
    assert lib.lib.fastmax_normalize_backward_stats_bytes(C.byref(nd)) == 4 * 4 * (4 + 2 * 64 + 4 + 2 * 2)
    # forward: 2 header floats, the token mean, one maximum per 256 tokens (+ column sums per 256 tokens), even count
    assert lib.lib.fastmax_normalize_stats_bytes(C.byref(nd)) == 4 * 4 * (2 + 64 + 1 + 1)
    nd.centre, nd.n = 2, 600
    assert lib.lib.fastmax_normalize_stats_bytes(C.byref(nd)) == 4 * 4 * (2 + 64 + 3 + 3 * 64 + 1)
    assert lib.lib.fastmax_normalize_stats_bytes(None) == 0
    nd.n = 130
    assert lib.lib.fastmax_normalize_backward_stats_bytes(None) == 0
    one = C.c_void_p(256)     # never dereferenced: validation fails first
    assert lib.lib.fastmax_normalize_backward(C.byref(nd), None, one, one, one, None) == 1
    assert lib.lib.fastmax_normalize_backward(C.byref(nd), one, one, one, None, None) == 4   # needs its scratch
    nd.d = 48
    assert lib.lib.fastmax_normalize_backward(C.byref(nd), one, one, one, one, None) == 3
    nd.d, nd.centre = 64, 5
    assert lib.lib.fastmax_normalize_backward(C.byref(nd), one, one, one, one, None) == 3

