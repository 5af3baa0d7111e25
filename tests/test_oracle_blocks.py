"""Pins oracle/blocks.py (the element-wise block steps): hand-computed rows, library routines in float64, and
orderings of the steps that a transposed or dropped operation would break."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import blocks


def test_layernorm_row_by_hand_and_against_torch():
    # row [1,2,3,4]: mean 2.5, biased variance 1.25
    a = np.array([[1.0, 2.0, 3.0, 4.0]])
    w = np.array([1.0, 2.0, 3.0, 4.0])
    b = np.array([0.5, 0.0, -0.5, 1.0])
    want = (a[0] - 2.5) / np.sqrt(1.25 + 1e-5) * w + b
    got = blocks.row_epilogue(a, None, w, b, None, blocks.PRE_NONE, blocks.POST_NONE, 1e-5)
    assert np.allclose(got[0], want, rtol=0, atol=1e-15)
    rng = np.random.default_rng(0)
    a = rng.standard_normal((3, 5, 24)) * 3 + 1
    w, b = rng.standard_normal(24), rng.standard_normal(24)
    ref = F.layer_norm(torch.from_numpy(a), (24,), torch.from_numpy(w), torch.from_numpy(b), 1e-5).numpy()
    assert np.allclose(blocks.row_epilogue(a, None, w, b), ref, rtol=0, atol=1e-13)


def test_relu_square_comes_before_the_norm_and_the_gate_after():
    a = np.array([[-1.0, 2.0, -3.0, 1.0]])
    # relu^2 -> [0, 4, 0, 1]
    assert np.array_equal(blocks.row_epilogue(a, pre=blocks.PRE_RELU_SQ), [[0.0, 4.0, 0.0, 1.0]])
    other = np.array([[0.0, 0.0, np.log(3.0), -np.log(3.0)]])       # sigmoid: 0.5, 0.5, 0.75, 0.25
    got = blocks.row_epilogue(a, other, pre=blocks.PRE_RELU_SQ, post=blocks.POST_SIGMOID_GATE)
    assert np.allclose(got, [[0.0, 2.0, 0.0, 0.25]], rtol=0, atol=1e-15)
    # with LayerNorm in between: mean 1.25, var (1.5625 + 7.5625 + 1.5625 + 0.0625)/4 = 2.6875
    w, b = np.ones(4), np.zeros(4)
    got = blocks.row_epilogue(a, other, w, b, None, blocks.PRE_RELU_SQ, blocks.POST_SIGMOID_GATE, 0.0)
    y = (np.array([0.0, 4.0, 0.0, 1.0]) - 1.25) / np.sqrt(2.6875)
    assert np.allclose(got[0], y * np.array([0.5, 0.5, 0.75, 0.25]), rtol=0, atol=1e-15)


def test_residual_with_and_without_layer_scale():
    a = np.array([[1.0, -2.0]])
    x = np.array([[10.0, 20.0]])
    g = np.array([0.5, 2.0])
    assert np.array_equal(blocks.row_epilogue(a, x, post=blocks.POST_RESIDUAL), [[11.0, 18.0]])
    assert np.array_equal(blocks.row_epilogue(a, x, gamma=g, post=blocks.POST_RESIDUAL), [[10.5, 16.0]])
    # post-norm block: x + gamma * ln(a); a row of two values normalises to -1, +1 (eps = 0)
    got = blocks.row_epilogue(a, x, np.ones(2), np.zeros(2), g, blocks.PRE_NONE, blocks.POST_RESIDUAL, 0.0)
    assert np.allclose(got, [[10.0 + 0.5 * 1.0, 20.0 + 2.0 * -1.0]], rtol=0, atol=1e-15)


def test_maa_mix_by_hand():
    x = np.array([[1.0, 2.0]])
    sx = np.array([[3.0, -2.0]])                                   # xx = [2, -4]
    m = np.stack([np.full((1, 2), 0.1 * i) for i in range(5)])
    maas = [np.array([0.5, 0.25])] * 5
    got = blocks.maa_mix(x, sx, m, maas)
    for i in range(5):
        assert np.allclose(got[i], [[1.0 + 2.0 * (0.5 + 0.1 * i), 2.0 - 4.0 * (0.25 + 0.1 * i)]], rtol=0, atol=1e-15)
    # maa + m = 1 gives the shifted input, 0 gives x
    assert np.array_equal(blocks.maa_mix(x, sx, np.zeros((5, 1, 2)), [np.ones(2)] * 5)[3], sx)
    assert np.array_equal(blocks.maa_mix(x, sx, np.zeros((5, 1, 2)), [np.zeros(2)] * 5)[0], x)


def test_groupnorm_gate_against_torch_and_by_hand():
    rng = np.random.default_rng(1)
    y = rng.standard_normal((2, 3, 16)) * 2 + 0.5
    gate = rng.standard_normal((2, 3, 16))
    w, b = rng.standard_normal(16), rng.standard_normal(16)
    t = torch.from_numpy
    ref = F.group_norm(t(y).reshape(-1, 16), 4, t(w), t(b), 1e-5).view(2, 3, 16) * F.silu(t(gate))
    assert np.allclose(blocks.groupnorm_gate(y, gate, w, b, 4), ref.numpy(), rtol=0, atol=1e-13)
    # one token, two groups of two channels: each group normalises to (-1, +1); silu(0) = 0, silu(large) -> identity
    got = blocks.groupnorm_gate(np.array([[1.0, 3.0, 10.0, 20.0]]), np.array([[0.0, 40.0, 40.0, 40.0]]),
                                np.array([1.0, 2.0, 3.0, 4.0]), np.array([0.0, 1.0, 0.0, -1.0]), 2, eps=0.0)
    assert np.allclose(got, [[0.0, 40.0 * 3.0, 40.0 * -3.0, 40.0 * 3.0]], rtol=1e-12, atol=0)
