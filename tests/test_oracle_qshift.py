import numpy as np

from conftest import load_golden
from oracle import qshift


def _slices(x, s, g, Hp, Wp):
    """Tensor-slicing restatement (independent of the index loops)."""
    B, T, C = x.shape
    a = x.transpose(0, 2, 1).reshape(B, C, Hp, Wp)
    o = np.zeros_like(a)
    o[:, 0:g, :, s:] = a[:, 0:g, :, :Wp - s]
    o[:, g:2 * g, :, :Wp - s] = a[:, g:2 * g, :, s:]
    o[:, 2 * g:3 * g, s:, :] = a[:, 2 * g:3 * g, :Hp - s, :]
    o[:, 3 * g:4 * g, :Hp - s, :] = a[:, 3 * g:4 * g, s:, :]
    o[:, 4 * g:] = a[:, 4 * g:]
    return o.reshape(B, C, T).transpose(0, 2, 1)


def test_loops_vs_slices_and_borders():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 4 * 6, 18))
    y = qshift.q_shift_loops(x, 1, 0.25, (4, 6))
    g = int(18 * 0.25)
    assert np.array_equal(y, _slices(x, 1, g, 4, 6))
    yg = y.reshape(2, 4, 6, 18)
    assert (yg[:, :, 0, 0:g] == 0).all() and (yg[:, :, -1, g:2 * g] == 0).all()
    assert (yg[:, 0, :, 2 * g:3 * g] == 0).all() and (yg[:, -1, :, 3 * g:4 * g] == 0).all()
    assert np.array_equal(y[..., 4 * g:], x[..., 4 * g:])


def test_multihead_equals_per_head_qshift():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, 3 * 4, 16))
    y = qshift.q_shift_multihead_loops(x, 1, 8, (3, 4))
    for h in range(2):
        want = qshift.q_shift_loops(x[..., 8 * h:8 * h + 8], 1, 0.25, (3, 4))
        assert np.array_equal(y[..., 8 * h:8 * h + 8], want)
    xc = np.concatenate([x, rng.standard_normal((1, 1, 16))], axis=1)
    yc = qshift.q_shift_multihead_loops(xc, 1, 8, (3, 4), with_cls_token=True)
    assert np.array_equal(yc[:, :-1], y) and np.array_equal(yc[:, -1], xc[:, -1])


def test_golden():
    g = load_golden("qshift_golden")
    assert np.array_equal(qshift.q_shift_loops(g["q"]["x"], 1, 0.25, (3, 5)), g["q"]["y"])
    assert np.array_equal(qshift.q_shift_multihead_loops(g["mh"]["x"], 1, 8, (4, 3), True), g["mh"]["y"])
