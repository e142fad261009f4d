"""Host-side view algebra (arraymancer_amd/metadata.py) against NumPy's own strided views and the
reference's explicit-broadcast vectors — CPU only."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from arraymancer_amd import metadata as md
from arraymancer_amd.metadata import Layout, Step


def np_layout(v: np.ndarray, base: np.ndarray) -> Layout:
    it = v.dtype.itemsize
    off = (v.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // it
    return Layout(tuple(v.shape), tuple(s // it for s in v.strides), off)


def test_shape_to_strides():
    assert md.shape_to_strides((3, 5)) == (5, 1)
    assert md.shape_to_strides((3, 5), "F") == (1, 3)
    assert md.shape_to_strides((2, 3, 4)) == (12, 4, 1)
    with pytest.raises(ValueError):
        md.contiguous((1,) * 7)


def test_transpose_and_contiguity():
    l = md.contiguous((4, 6))
    t = md.transpose(l)
    assert t.shape == (6, 4) and t.strides == (1, 6)
    assert md.is_C_contiguous(l) and not md.is_F_contiguous(l)
    assert md.is_F_contiguous(t) and not md.is_C_contiguous(t)
    # strides of extent-1 axes are ignored
    assert md.is_C_contiguous(Layout((1, 5), (77, 1)))
    assert md.is_C_contiguous(Layout((5, 1), (1, 99)))


def test_reference_slices():
    """The exact slices of test_operators_blas.nim:347-365 and :157-193."""
    base = np.arange(24).reshape(6, 4)
    l = md.contiguous((6, 4))
    assert md.slicer(l, [Step(4, 2, -2), Step(3, 1, -2)]) == np_layout(base[4:1:-2, 3:0:-2], base)
    assert md.slicer(l, [Step(2, 3, 1), Step(3, 1, -2)]) == np_layout(base[2:4, 3:0:-2], base)
    f = md.contiguous((2, 2), "F")
    s = md.slicer(f, [Step(0, 1, 1), Step(1, 0, -1, a_from_end=True)])     # [_, ^1..0|-1]
    assert s.shape == (2, 2) and s.strides == (1, -2) and s.offset == 2
    with pytest.raises(IndexError):
        md.slicer(l, [Step(0, 6, 1)])
    with pytest.raises(IndexError):
        md.slicer(l, [Step(0, 1, 1)] * 3)
    with pytest.raises(IndexError):
        md.slicer(l, [Step(3, 1, 1)])


@settings(max_examples=200, deadline=None)
@given(st.lists(st.integers(1, 6), min_size=1, max_size=4), st.data())
def test_python_indexing_matches_numpy(shape, data):
    base = np.arange(int(np.prod(shape))).reshape(shape)
    key = []
    for n in shape:
        kind = data.draw(st.sampled_from(["all", "slice", "int"]))
        if kind == "all":
            key.append(slice(None))
        elif kind == "int":
            key.append(data.draw(st.integers(-n, n - 1)))
        else:
            step = data.draw(st.sampled_from([1, 2, 3, -1, -2]))
            a = data.draw(st.one_of(st.none(), st.integers(-n, n)))
            b = data.draw(st.one_of(st.none(), st.integers(-n, n)))
            key.append(slice(a, b, step))
    got = md.py_index(md.contiguous(shape), tuple(key))
    npkey = tuple(slice(k, k + 1 if k != -1 else None) if isinstance(k, int) else k for k in key)
    want = base[npkey]
    assert got.shape == want.shape
    if want.size:
        lw = np_layout(want, base)
        # element addresses must coincide wherever the extent is > 1
        assert got.offset == lw.offset
        assert all(g == w for g, w, n in zip(got.strides, lw.strides, got.shape) if n > 1)


def test_broadcast_reference_vectors(vectors):
    for case in vectors["explicit_broadcast"]:
        t = np.array(case["t"])
        l = md.broadcast(md.contiguous(t.shape), case["shape"])
        v = np.lib.stride_tricks.as_strided(t, shape=l.shape, strides=tuple(s * t.itemsize for s in l.strides))
        assert np.array_equal(v, np.array(case["expect"]))


def test_broadcast_rules():
    a, b = md.contiguous((4, 1)), md.contiguous((1, 3))
    ba, bb = md.broadcast2(a, b)
    assert ba.shape == bb.shape == (4, 3) and ba.strides == (1, 0) and bb.strides == (0, 1)
    with pytest.raises(ValueError):
        md.broadcast2(md.contiguous((4, 2)), md.contiguous((1, 3)))
    with pytest.raises(ValueError):
        md.broadcast2(md.contiguous((4,)), md.contiguous((1, 3)))
    with pytest.raises(ValueError):
        md.broadcast(md.contiguous((4, 2)), (4, 3))
    # scalar broadcast: one element, all strides zero (shapeshifting.nim:151-155)
    s = md.broadcast(md.contiguous((1, 1)), (3, 2))
    assert s.strides == (0, 0) and s.size == 6


def test_extent_in_storage():
    assert md.extent_in_storage(Layout((2, 2), (-8, -2), 19)) == (9, 19)
    assert md.extent_in_storage(Layout((3, 4), (4, 1), 0)) == (0, 11)
    assert md.extent_in_storage(Layout((0, 4), (4, 1), 5)) == (5, 4)


def test_permute_squeeze_unsqueeze_match_numpy():
    """permute / squeeze / unsqueeze (shapeshifting.nim:207-226, 396-424) are metadata only: the same elements as the
    NumPy view of the same name, and unsqueeze's new stride is the reference's shape[axis] * strides[axis]."""
    from arraymancer_amd import metadata as md
    base = np.arange(2 * 1 * 3 * 1 * 4).reshape(2, 1, 3, 1, 4)

    def view(l):
        return np.lib.stride_tricks.as_strided(base.reshape(-1)[l.offset:], shape=l.shape, strides=tuple(s * base.itemsize for s in l.strides))

    l = md.contiguous(base.shape)
    assert np.array_equal(view(md.permute(l, (4, 2, 0, 1, 3))), base.transpose(4, 2, 0, 1, 3))
    with pytest.raises(ValueError):
        md.permute(l, (0, 1, 2, 3, 3))
    assert np.array_equal(view(md.squeeze(l)), base.squeeze())
    assert np.array_equal(view(md.squeeze(l, 1)), base.squeeze(1))
    assert md.squeeze(l, 0) == l                                      # extent 2: nothing to drop
    ones = md.contiguous((1, 1))
    assert md.squeeze(ones).shape == (1,)                             # the rank never drops to 0
    u = md.unsqueeze(md.contiguous((3, 4)), 1)
    assert u.shape == (3, 1, 4) and u.strides == (4, 4, 1)
    assert md.unsqueeze(md.contiguous((3, 4)), 2).strides == (4, 1, 1)
    assert np.array_equal(view(md.unsqueeze(md.squeeze(l), 0))[0], base.squeeze())
