import numpy as np

from conftest import load_golden
from oracle import qshift


def _slices(x, s, bounds, Hp, Wp):
    """Tensor-slicing restatement (independent of the index loops); `bounds` are the upper ends of the four
    shifted channel groups, stated by hand in each test."""
    B, T, C = x.shape
    b1, b2, b3, b4 = bounds
    a = x.transpose(0, 2, 1).reshape(B, C, Hp, Wp)
    o = np.zeros_like(a)
    o[:, 0:b1, :, s:] = a[:, 0:b1, :, :Wp - s]
    o[:, b1:b2, :, :Wp - s] = a[:, b1:b2, :, s:]
    o[:, b2:b3, s:, :] = a[:, b2:b3, :Hp - s, :]
    o[:, b3:b4, :Hp - s, :] = a[:, b3:b4, s:, :]
    o[:, b4:] = a[:, b4:]
    return o.reshape(B, C, T).transpose(0, 2, 1)


def test_loops_vs_slices_and_borders():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 4 * 6, 16))
    y = qshift.q_shift_loops(x, 1, 0.25, (4, 6))
    g = 4
    assert np.array_equal(y, _slices(x, 1, (4, 8, 12, 16), 4, 6))
    yg = y.reshape(2, 4, 6, 16)
    assert (yg[:, :, 0, 0:g] == 0).all() and (yg[:, :, -1, g:2 * g] == 0).all()
    assert (yg[:, 0, :, 2 * g:3 * g] == 0).all() and (yg[:, -1, :, 3 * g:4 * g] == 0).all()
    # gamma < 1/4 leaves pass-through channels: 20 * 0.2 -> groups of 4, channels 16..19 copied
    x = rng.standard_normal((1, 3 * 4, 20))
    y = qshift.q_shift_loops(x, 1, 0.2, (3, 4))
    assert np.array_equal(y, _slices(x, 1, (4, 8, 12, 16), 3, 4))
    assert np.array_equal(y[..., 16:], x[..., 16:])


def test_unequal_channel_groups():
    """C*gamma not an integer: the reference cuts at int(C*gamma*k) (vrwkv.py:72-76), so the groups are unequal and
    nothing passes through -- C=18: 0,4,9,13,18; C=22: 0,5,11,16,22; C=6: 0,1,3,4,6 (worked out by hand)."""
    rng = np.random.default_rng(5)
    for C, bounds in ((18, (4, 9, 13, 18)), (22, (5, 11, 16, 22)), (6, (1, 3, 4, 6))):
        x = rng.standard_normal((2, 3 * 5, C))
        y = qshift.q_shift_loops(x, 1, 0.25, (3, 5))
        assert np.array_equal(y, _slices(x, 1, bounds, 3, 5)), C
        yg, xg = y.reshape(2, 3, 5, C), x.reshape(2, 3, 5, C)
        b1, b2, b3, b4 = bounds
        # last channel of the second group moves left, first channel of the third group moves down
        assert np.array_equal(yg[:, :, :-1, b2 - 1], xg[:, :, 1:, b2 - 1]) and (yg[:, :, -1, b2 - 1] == 0).all()
        assert np.array_equal(yg[:, 1:, :, b2], xg[:, :-1, :, b2]) and (yg[:, 0, :, b2] == 0).all()
        assert b4 == C


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
