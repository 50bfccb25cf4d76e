"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares,
and rejects bad descriptors / pointers / workspaces before anything reaches a device."""
import ctypes as C
import os
import re

import pytest

from fastmax_amd import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = 0x10000  # a non-NULL pointer that is never dereferenced: validation fails first


def desc(**over):
    base = dict(bh=4, n=100, d=64, dtype=_cabi.FASTMAX_F32, mask=True, normalize=True, p=2)
    base.update(over)
    return _cabi.make_desc(**base)


def test_exports_match_header(built):
    text = open(os.path.join(ROOT, "include", "fastmax_amd.h")).read()
    declared = set(re.findall(r"\b(fastmax_[a-z_]+)\s*\(", text))
    assert declared == set(_cabi.EXPORTS)
    for name in declared:
        assert getattr(built, name) is not None


def test_version_and_clean_error(built):
    assert built.fastmax_version().decode() == "0.1"
    assert built.fastmax_check_desc(C.byref(desc())) == 0
    assert _cabi.last_error() == ""


@pytest.mark.parametrize("over,code", [
    (dict(d=50), -2), (dict(d=132), -2), (dict(d=0), -2), (dict(d=12, dtype=1), -2), (dict(bh=0), -2), (dict(bhkv=3), -2), (dict(bhkv=0), -2), (dict(nk=50), -2), (dict(n=0), -2),
    (dict(dtype=7), -3), (dict(p=3), -4), (dict(p=0), -4), (dict(lim=0.0), -4),
    (dict(normalize=False, temperature=0.0), -4),
])
def test_bad_descriptors(built, over, code):
    assert built.fastmax_check_desc(C.byref(desc(**over))) == code
    assert _cabi.last_error() != ""
    assert built.fastmax_workspace_bytes(C.byref(desc(**over)), _cabi.PASS_FORWARD) == 0


def test_head_dimensions_and_the_dense_plan(built, monkeypatch):
    """Any head dimension that is a whole number of 16-byte pieces up to 128 is served (the reference's
    launcher reads d at run time, fastmax_cuda_forward.cu:331-338): dimensions other than 32 and 64 by
    the dense score-tile kernels, which keep no states -- the workspace holds the per-head scalars (and,
    backward, c_i and the normalisation partials) only.  Left to itself the library also takes those
    kernels for short sequences at d = 32 / 64; the recurrent entry points keep moment states and so
    stay with d = 32 / 64."""
    for d, dtype in ((4, 0), (16, 0), (48, 0), (96, 0), (128, 0), (8, 1), (48, 1), (128, 1)):
        ds = desc(d=d, dtype=dtype, bh=6, n=5000, mask=True)
        assert built.fastmax_check_desc(C.byref(ds)) == 0, _cabi.last_error()
        assert built.fastmax_workspace_bytes(C.byref(ds), _cabi.PASS_FORWARD) == 512
        assert built.fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_BACKWARD) == \
            512 + (6 * 5000 * 4 + 255) // 256 * 256 + (6 * 2 * 40 * 4 + 255) // 256 * 256
        assert built.fastmax_saved_state_bytes(C.byref(ds)) == 256
        assert built.fastmax_state_bytes(C.byref(ds)) == 0 and "recurrent" in _cabi.last_error()
    # p = 1 past 1024 causal / 512 unmasked positions: the dense kernels take one small state per 256 positions
    # with them (linear time): per key/value head and slot the d x d block in one layout plus the sums,
    # backward also per query head the block in both layouts
    a256 = lambda x: (x + 255) // 256 * 256
    r64 = lambda x: (x + 63) // 64 * 64
    for d, dp in ((128, 128), (48, 64), (80, 96)):
        one, two = r64(dp * (dp + 4) + 2 * dp + 4), r64(2 * dp * (dp + 4) + 2 * dp + 4)
        ds = desc(d=d, dtype=0, bh=6, bhkv=3, n=5000, mask=True, p=1)
        assert built.fastmax_workspace_bytes(C.byref(ds), _cabi.PASS_FORWARD) == 512 + a256(3 * 20 * one * 4)
        assert built.fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_BACKWARD) == \
            512 + a256(6 * 5000 * 4) + a256(6 * 2 * 40 * 4) + a256(3 * 20 * one * 4) + a256(6 * 20 * two * 4)
        assert built.fastmax_saved_state_bytes(C.byref(ds)) == 256
        assert built.fastmax_workspace_bytes(C.byref(desc(d=d, bh=6, n=1000, mask=True, p=1)), _cabi.PASS_FORWARD) == 512
        assert built.fastmax_workspace_bytes(C.byref(desc(d=d, bh=6, n=600, mask=False, p=1)), _cabi.PASS_FORWARD) == \
            512 + a256(6 * 3 * one * 4)
    short, long_ = desc(bh=96, n=2048, dtype=1, mask=True), desc(bh=96, n=16384, dtype=1, mask=True)
    assert built.fastmax_workspace_bytes(C.byref(short), _cabi.PASS_FORWARD) > 1 << 20   # (FASTMAX_PATH=moments here)
    monkeypatch.delenv("FASTMAX_PATH")
    assert built.fastmax_workspace_bytes(C.byref(short), _cabi.PASS_FORWARD) == 1536
    assert built.fastmax_workspace_bytes(C.byref(long_), _cabi.PASS_FORWARD) > 1 << 20
    assert built.fastmax_workspace_bytes(C.byref(desc(bh=96, n=2048, dtype=1, mask=True, p=1)), _cabi.PASS_FORWARD) > 1 << 20
    monkeypatch.setenv("FASTMAX_PATH", "dense")
    assert built.fastmax_workspace_bytes(C.byref(long_), _cabi.PASS_FORWARD) == 1536


def test_kernel_choice_for_p1(built, monkeypatch):
    """p = 1 at d = 32 / 64 stays with the moment kernels except for bf16 inputs under the mask past 1024 keys
    when the one-scan-per-head kernels are not there to take them (d = 64, ungrouped heads, no key prefix,
    at least 208 heads with bf16 tensors): then the dense kernels' linear mode runs."""
    monkeypatch.delenv("FASTMAX_PATH")
    uses = lambda **kw: built.fastmax_uses_dense_tiles(C.byref(desc(p=1, **kw)))
    assert uses(bh=96, n=2048, dtype=1, mask=True) == 1
    assert uses(bh=207, n=4096, dtype=1, mask=True) == 1
    assert uses(bh=208, n=4096, dtype=1, mask=True) == 0
    assert uses(bh=512, n=16384, dtype=1, mask=True) == 0
    assert uses(bh=1024, n=10000, dtype=1, mask=True) == 0
    assert uses(bh=1024, bhkv=256, n=4096, dtype=1, mask=True) == 1   # (grouped heads: no scan kernels)
    assert uses(bh=1024, n=4096, d=32, dtype=1, mask=True) == 1       # (d = 32: no scan kernels)
    assert uses(bh=1024, n=4096, nk=5000, dtype=1, mask=True) == 1    # (a key prefix: no scan kernels)
    assert uses(bh=96, n=1024, dtype=1, mask=True) == 0
    assert uses(bh=96, n=2048, dtype=1, mask=False) == 0
    assert uses(bh=96, n=2048, dtype=0, mask=True) == 0
    assert uses(bh=96, n=2048, d=48, dtype=0, mask=True) == 1
    # the scan kernels keep no states: with bf16 tensors from 208 heads on, with fp32 tensors from 512
    tiny = lambda **kw: built.fastmax_workspace_bytes(C.byref(desc(p=1, mask=True, n=1000, **kw)), _cabi.PASS_FORWARD)
    assert tiny(bh=208, dtype=1) == 2 * 256 * ((208 * 8 + 255) // 256) and tiny(bh=207, dtype=1) > 1 << 16
    assert tiny(bh=511, dtype=0) > 1 << 16


def test_kernel_choice_for_p2(built, monkeypatch):
    """p = 2 at d = 32 / 64: the dense score tiles up to the measured crossover (key counts; the first figure
    of a pair is for at most 128 heads), the moment kernels beyond; a causal sequence of a single chunk stays
    with the moment kernels; other head dimensions have dense kernels only."""
    monkeypatch.delenv("FASTMAX_PATH")
    uses = lambda **kw: built.fastmax_uses_dense_tiles(C.byref(desc(p=2, **kw)))
    table = [  # d, dtype (0 fp32, 1 bf16), mask, limit with few heads, limit with many
        (64, 1, True, 5632, 4096), (64, 1, False, 2048, 1536), (64, 0, True, 3584, 3072), (64, 0, False, 1024, 1024),
        (32, 1, True, 3072, 2048), (32, 1, False, 1024, 768), (32, 0, True, 1536, 1024), (32, 0, False, 512, 512),
    ]
    for d, dtype, mask, few, many in table:
        for bh, limit in ((96, few), (128, few), (129, many), (768, many)):
            assert uses(d=d, dtype=dtype, mask=mask, bh=bh, n=limit) == 1, (d, dtype, mask, bh, limit)
            assert uses(d=d, dtype=dtype, mask=mask, bh=bh, n=limit + 1) == 0, (d, dtype, mask, bh, limit)
    # a single causal chunk (384 positions for bf16, 256 for fp32 at d = 64, 128 at d = 32)
    assert uses(d=64, dtype=1, mask=True, bh=96, n=384) == 0 and uses(d=64, dtype=1, mask=True, bh=96, n=385) == 1
    assert uses(d=64, dtype=0, mask=True, bh=96, n=256) == 0 and uses(d=64, dtype=0, mask=True, bh=96, n=257) == 1
    assert uses(d=32, dtype=0, mask=True, bh=96, n=128) == 0 and uses(d=32, dtype=0, mask=True, bh=96, n=129) == 1
    assert uses(d=64, dtype=1, mask=False, bh=96, n=32) == 1
    # the configurations of the benchmark: 1 and 3 (headline) and 4 on the moment kernels, 2 and 5 on the dense ones
    assert uses(d=32, dtype=0, mask=False, bh=64, n=1024) == 0
    assert uses(d=32, dtype=0, mask=True, bh=512, n=1000) == 1
    assert uses(d=64, dtype=0, mask=True, bh=1024, n=10000) == 0
    assert uses(d=64, dtype=1, mask=True, bh=512, n=16384) == 0
    assert uses(d=64, dtype=1, mask=True, bh=96, n=2048) == 1
    for d in (16, 48, 96, 128):
        assert uses(d=d, dtype=0, mask=True, bh=4, n=20000) == 1


def test_grouped_heads_descriptor(built):
    """bhkv must divide bh (fastmax_cuda_forward.cu:38 maps head i to key/value head i / (bh/bhkv)); the
    smallest workspace then holds one whole group."""
    ds1, ds4 = desc(bh=8, bhkv=8, mask=True), desc(bh=8, bhkv=2, mask=True)
    assert built.fastmax_check_desc(C.byref(ds4)) == 0
    for pas in (_cabi.PASS_FORWARD, _cabi.PASS_BACKWARD):
        lo1 = built.fastmax_workspace_min_bytes(C.byref(ds1), pas)
        lo4 = built.fastmax_workspace_min_bytes(C.byref(ds4), pas)
        assert lo4 > lo1 > 0


def test_bad_p_message_matches_reference_wording(built):
    # the reference raises ValueError(f"p must be 1 or 2, got: {p}") (example.py:195-196)
    built.fastmax_check_desc(C.byref(desc(p=5)))
    assert _cabi.last_error() == "p must be 1 or 2, got: 5"


def test_null_desc(built):
    assert built.fastmax_check_desc(None) == -1


def test_workspace_sizes(built):
    for mask in (False, True):
        for pas in (_cabi.PASS_FORWARD, _cabi.PASS_BACKWARD):
            ds = desc(bh=1024, n=10000, mask=mask)
            lo = built.fastmax_workspace_min_bytes(C.byref(ds), pas)
            hi = built.fastmax_workspace_bytes(C.byref(ds), pas)
            assert 0 < lo <= hi
            assert hi <= (16 << 30) + lo
    # causal d=64 p=2 fp32: one state is (33*64 + 64 + 1) rows of 68 floats, one per 256-token chunk
    ds = desc(bh=1, n=1000, mask=True)
    state = ((33 * 64 + 65) * 68 + 63) // 64 * 64 * 4
    assert built.fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_FORWARD) == 512 + 4 * state
    assert built.fastmax_workspace_bytes(C.byref(ds), 9) == 0  # unknown pass


def test_scan_path_needs_no_state_memory(built):
    """Causal p = 1, d = 64, >= 512 heads, n >= 32, a1 != 0 runs as one register-resident scan
    per head: the workspace holds only the per-head and per-token scalars."""
    ds = desc(bh=1024, n=10000, mask=True, p=1)
    fwd = built.fastmax_workspace_bytes(C.byref(ds), _cabi.PASS_FORWARD)
    bwd = built.fastmax_workspace_bytes(C.byref(ds), _cabi.PASS_BACKWARD)
    assert fwd == built.fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_FORWARD) == 2 * 4096 * 2
    blocks = (10000 + 127) // 128
    assert bwd == 2 * 8192 + 1024 * 10000 * 4 + 2 * 1024 * blocks * 4
    assert built.fastmax_saved_state_bytes(C.byref(ds)) == 256
    for other in (desc(bh=511, n=10000, mask=True, p=1), desc(bh=1024, n=31, mask=True, p=1),
                  desc(bh=1024, n=10000, mask=True, p=1, a1=0.0), desc(bh=1024, n=10000, mask=False, p=1)):
        assert built.fastmax_workspace_min_bytes(C.byref(other), _cabi.PASS_FORWARD) > 2 * 8192


def test_forward_rejects_before_touching_device(built):
    ds = desc()
    f = built.fastmax_forward
    assert f(C.byref(ds), None, FAKE, FAKE, FAKE, 64, FAKE, 1, None, None, FAKE, 1 << 30, None) == -1
    assert f(C.byref(ds), FAKE, FAKE, FAKE, FAKE, 63, FAKE, 1, None, None, FAKE, 1 << 30, None) == -4  # ldo < d
    assert f(C.byref(ds), FAKE, FAKE, FAKE, FAKE, 64, FAKE, 0, None, None, FAKE, 1 << 30, None) == -4  # den stride
    assert f(C.byref(ds), FAKE, FAKE, FAKE, FAKE, 64, FAKE, 1, None, None, None, 1 << 30, None) == -5
    assert f(C.byref(ds), FAKE, FAKE, FAKE, FAKE, 64, FAKE, 1, None, None, FAKE + 4, 1 << 30, None) == -5  # alignment
    assert f(C.byref(ds), FAKE, FAKE, FAKE, FAKE, 64, FAKE, 1, None, None, FAKE, 16, None) == -5  # too small
    assert "minimum" in _cabi.last_error()


def test_backward_rejects_before_touching_device(built):
    ds = desc()
    b = built.fastmax_backward
    args = [FAKE] * 3 + [FAKE, 64, FAKE, 1, FAKE, FAKE, FAKE, FAKE, None, None]
    assert b(C.byref(ds), *args, FAKE, 16, None) == -5
    args[0] = None
    assert b(C.byref(ds), *args, FAKE, 1 << 30, None) == -1
    assert built.fastmax_normalize_inplace(C.byref(ds), None, FAKE, FAKE, 1 << 20, None) == -1
    assert built.fastmax_normalize_inplace(C.byref(ds), FAKE, FAKE, FAKE, 8, None) == -5


def test_profile_end_without_launches(built):
    kt = _cabi.KernelTimes()
    assert built.fastmax_profile_begin() == 0
    assert built.fastmax_profile_end(C.byref(kt)) == 0
    assert sum(kt.launches) == 0
    assert built.fastmax_profile_end(None) == -1
