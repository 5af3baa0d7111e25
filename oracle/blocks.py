"""CPU restatement (NumPy float64) of the element-wise steps a VRWKV / VRWKV6 block runs around the WKV operators.
TEST INFRASTRUCTURE ONLY: imported by tests/, never by the operator path.

Each function restates, row by row, a short PyTorch-op sequence of the reference:
  row_epilogue      classification/mmcls_custom/models/backbones/vrwkv.py:184-186 (key_norm, sr * x),
                    :256-261 (relu^2, key_norm, sigmoid gate), :300-313 (x + gamma * ln(...), or without ln)
  maa_mix           .../vrwkv6.py:178-194  (xx = shift(x) - x;  x + xx * (time_maa_i + m_i), i = w, k, v, r, g)
  groupnorm_gate    .../vrwkv6.py:199, 205-211  (ln_x = GroupNorm(n_head, C) on the (B*T, C) view, times silu(gate))

Pinned by tests/test_oracle_blocks.py: hand-computed rows, LayerNorm / GroupNorm against torch.nn.functional in
float64 on the CPU, and the gate / residual algebra on values chosen so that a wrong order of the steps shows.
"""
import numpy as np

PRE_NONE, PRE_RELU_SQ = 0, 1
POST_NONE, POST_SIGMOID_GATE, POST_RESIDUAL = 0, 1, 2


def _layer_norm_row(row, weight, bias, eps):
    mean = row.sum() / row.size
    var = ((row - mean) ** 2).sum() / row.size          # biased variance, as torch.nn.LayerNorm
    return (row - mean) / np.sqrt(var + eps) * weight + bias


def row_epilogue(a, other=None, ln_weight=None, ln_bias=None, gamma=None, pre=PRE_NONE, post=POST_NONE, eps=1e-5):
    """out = post(LayerNorm(pre(a))) per row of the last axis; LayerNorm only when ln_weight is given."""
    a = np.asarray(a, np.float64)
    N = a.shape[-1]
    rows = a.reshape(-1, N)
    oth = None if other is None else np.asarray(other, np.float64).reshape(-1, N)
    out = np.empty_like(rows)
    for i in range(rows.shape[0]):
        y = rows[i]
        if pre == PRE_RELU_SQ:
            y = np.where(y > 0, y, 0.0) ** 2                                   # torch.square(torch.relu(k)), vrwkv.py:256
        if ln_weight is not None:
            y = _layer_norm_row(y, np.asarray(ln_weight, np.float64), np.asarray(ln_bias, np.float64), eps)
        if post == POST_SIGMOID_GATE:
            y = y / (1.0 + np.exp(-oth[i]))                                     # sigmoid(other) * y
        elif post == POST_RESIDUAL:
            y = oth[i] + (np.asarray(gamma, np.float64) * y if gamma is not None else y)
        out[i] = y
    return out.reshape(a.shape)


def maa_mix(x, sx, m, maas):
    """Five mixes x + (sx - x) * (maa_i + m_i); x, sx (..., C), m (5, ..., C), maas five (C,) vectors."""
    x = np.asarray(x, np.float64)
    xx = np.asarray(sx, np.float64) - x
    return [x + xx * (np.asarray(maa, np.float64).reshape(-1) + np.asarray(mi, np.float64))
            for maa, mi in zip(maas, m)]


def groupnorm_gate(y, gate, weight, bias, n_groups, eps=1e-5):
    """GroupNorm over each of the n_groups blocks of consecutive channels of every token, affine per channel,
    times silu(gate)."""
    y = np.asarray(y, np.float64)
    C = y.shape[-1]
    assert C % n_groups == 0
    G = C // n_groups
    rows = y.reshape(-1, C)
    gt = np.asarray(gate, np.float64).reshape(-1, C)
    w = np.asarray(weight, np.float64)
    b = np.asarray(bias, np.float64)
    out = np.empty_like(rows)
    for i in range(rows.shape[0]):
        for h in range(n_groups):
            seg = rows[i, h * G:(h + 1) * G]
            mean = seg.sum() / G
            var = ((seg - mean) ** 2).sum() / G
            out[i, h * G:(h + 1) * G] = (seg - mean) / np.sqrt(var + eps) * w[h * G:(h + 1) * G] + b[h * G:(h + 1) * G]
        out[i] *= gt[i] / (1.0 + np.exp(-gt[i]))                               # silu
    return out.reshape(y.shape)
