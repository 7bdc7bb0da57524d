"""Layout arithmetic: the C ABI against the oracle and against the invariants the formulas fix."""
import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from oracle import gradpath as oracle
from rannc_amd import _lib


@pytest.mark.parametrize("numel,es,r,aligned,seg,src", [
    # worked examples of calcAlignedNumElems / doRegister (fp16: unit = 8 * R elements)
    (1000, 2, 8, 1024, 128, [128] * 7 + [104]),
    (100, 2, 8, 128, 16, [16, 16, 16, 16, 16, 16, 4, 0]),
    (1000, 2, 1, 1000, 1000, [1000]),
    (1001, 2, 1, 1008, 1008, [1001]),
    (10, 4, 4, 16, 4, [4, 4, 2, 0]),
    (0, 4, 2, 0, 0, [0, 0]),
    (1, 4, 1, 4, 4, [1]),
])
def test_worked_examples(numel, es, r, aligned, seg, src):
    a, s, offs, srcs = _lib.segment_layout(numel, es, r)
    assert (a, s, srcs) == (aligned, seg, src)
    lay = oracle.segment_layout(numel, es, r)
    assert (lay.aligned_size, lay.segment_size, list(lay.offsets), list(lay.src_sizes)) == (a, s, offs, srcs)


@settings(max_examples=400, deadline=None)
@given(numel=st.integers(0, 2 ** 40), es=st.sampled_from([2, 4]), r=st.integers(1, 64))
def test_segment_layout_invariants(numel, es, r):
    a, s, offs, srcs = _lib.segment_layout(numel, es, r)
    unit = 16 // es * r
    assert a % unit == 0 and 0 <= a - numel < unit
    assert a == _lib.aligned_numel(numel, es, r) == oracle.calc_aligned_num_elems(numel, es, r)
    assert s * r == a
    assert sum(srcs) == numel
    assert offs[0] == 0 and all(offs[i + 1] == offs[i] + srcs[i] for i in range(r - 1))
    assert all(0 <= x <= s for x in srcs)
    # only trailing ranks may be short
    short = [i for i, x in enumerate(srcs) if x < s]
    assert short == list(range(short[0], r)) if short else True
    lay = oracle.segment_layout(numel, es, r)
    assert list(lay.offsets) == offs and list(lay.src_sizes) == srcs


@settings(max_examples=200, deadline=None)
@given(items=st.lists(st.tuples(st.integers(0, 10 ** 9), st.sampled_from(["f32", "f16", "bf16"])), max_size=40))
def test_bucket_layout_matches_oracle_and_tiles(items):
    numels = [n for n, _ in items]
    names = [d for _, d in items]
    offs, lens = _lib.bucket_layout(numels, [_lib.DTYPE_CODES[d] for d in names])
    want_offs, want_lens = oracle.bucket_layout(numels, names)
    assert offs == want_offs
    for d, code in _lib.DTYPE_CODES.items():
        assert lens[code] == want_lens.get(d, 0)
        # views of one dtype tile their bucket exactly, in order, with no padding
        spans = [(o, o + n) for o, n, dd in zip(offs, numels, names) if dd == d]
        pos = 0
        for lo, hi in spans:
            assert lo == pos
            pos = hi
        assert pos == lens[code]
