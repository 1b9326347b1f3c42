"""View arithmetic of the Backend mirror (backend/view.go:23-165), on the CPU."""
import numpy as np

from mimir_amd.backend import View


def test_contiguous_shrink_permute_expand():
    v = View.contiguous([10, 1280])
    assert v.strides == [1280, 1] and v.offset == 0 and v.is_contiguous() and v.size() == 12800
    rows = v.shrink([(1, 10), (0, 1280)])
    assert rows.shape == [9, 1280] and rows.offset == 1280 and rows.is_contiguous()
    t = v.permute([1, 0])
    assert t.shape == [1280, 10] and t.strides == [1, 1280] and not t.is_contiguous()
    e = View.contiguous([3, 1]).expand([3, 7])
    assert e.strides == [1, 0] and e.shape == [3, 7]
    # an empty range keeps the offset (view.go: Shrink adds only for non-empty dimensions)
    assert v.shrink([(4, 4), (0, 1280)]).offset == 0
    # dimensions of one element do not count for contiguity
    assert View([1, 5], [99, 1]).is_contiguous() and View([5, 0], [7, 3]).is_contiguous() and not View([0, 5], [3, 7]).is_contiguous()


def test_indices_follow_strides():
    v = View.contiguous([4, 6]).permute([1, 0]).shrink([(1, 5), (0, 3)])
    base = np.arange(24).reshape(4, 6)
    assert np.array_equal(v.indices(), base.T[1:5, 0:3])
