"""CPU restatement (NumPy float64) of the element-wise steps a VRWKV / VRWKV6 block runs around the WKV operators.
TEST INFRASTRUCTURE ONLY: imported by tests/, never by the operator path.

Each function restates, row by row, a short PyTorch-op sequence of the reference:
  row_epilogue      classification/mmcls_custom/models/backbones/vrwkv.py:184-186 (key_norm, sr * x),
                    :256-261 (relu^2, key_norm, sigmoid gate), :300-313 (x + gamma * ln(...), or without ln)
  maa_mix           .../vrwkv6.py:178-194  (xx = shift(x) - x;  x + xx * (time_maa_i + m_i), i = w, k, v, r, g)
  groupnorm_gate    .../vrwkv6.py:199, 205-211  (ln_x = GroupNorm(n_head, C) on the (B*T, C) view, times silu(gate))

  spatial_mix, channel_mix, block   a whole VRWKV block composed of the above, the q_shift loops and an operator passed
                    in by the caller: .../vrwkv.py:156-188 (VRWKV_SpatialMix), :244-262 (VRWKV_ChannelMix),
                    :296-313 (Block: post- or pre-norm, with or without layer scale)
  spatial_mix_v6, block_v6          the VRWKV6 block: .../vrwkv6.py:175-228 (VRWKV_SpatialMix_V6: data-dependent mixes
                    and decay through the low-rank tanh bottlenecks, wkv6, key_norm, ln_x, silu gate, output),
                    :271-286 (its channel mix: the VRWKV one with the per-head shift), :314-332 (Block)

Pinned by tests/test_oracle_blocks.py: hand-computed rows, LayerNorm / GroupNorm against torch.nn.functional in
float64 on the CPU, the gate / residual algebra on values chosen so that a wrong order of the steps shows, and the
composed block against the same sequence written with torch float64 tensor ops and slice-copy shifts (every variant of
norm placement, layer scale and key_norm; identity-projection special cases by hand).
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


def _linear(x, weight):
    """nn.Linear without bias: x (..., in) times weight (out, in) transposed."""
    return np.asarray(x, np.float64) @ np.asarray(weight, np.float64).T


def _mix(x, xx, m):
    m = np.asarray(m, np.float64).reshape(1, 1, -1)
    return x * m + xx * (1.0 - m)                                         # vrwkv.py:161-163, 249-250


def spatial_mix(x, P, patch_resolution, wkv, shift_pixel=1, gamma=0.25, eps=1e-5):
    """VRWKV_SpatialMix.forward (vrwkv.py:156-188).  x (B,T,C); P: parameters by the reference's names
    (spatial_mix_k/v/r, key.weight, value.weight, receptance.weight, output.weight, spatial_decay, spatial_first and,
    with key_norm, key_norm.weight / key_norm.bias); wkv(w, u, k, v) -> y is the Bi-WKV operator to use."""
    from .qshift import q_shift_loops
    x = np.asarray(x, np.float64)
    B, T, C = x.shape
    xx = q_shift_loops(x, shift_pixel, gamma, patch_resolution) if shift_pixel > 0 else x
    xk, xv, xr = (_mix(x, xx, P[n]) if shift_pixel > 0 else x for n in ("spatial_mix_k", "spatial_mix_v", "spatial_mix_r"))
    k, v, r = _linear(xk, P["key.weight"]), _linear(xv, P["value.weight"]), _linear(xr, P["receptance.weight"])
    y = np.asarray(wkv(np.asarray(P["spatial_decay"], np.float64) / T, np.asarray(P["spatial_first"], np.float64) / T, k, v),
                   np.float64)                                            # vrwkv.py:183
    has_norm = "key_norm.weight" in P
    y = row_epilogue(y, r, P["key_norm.weight"] if has_norm else None, P["key_norm.bias"] if has_norm else None,
                     None, PRE_NONE, POST_SIGMOID_GATE, eps).reshape(B, T, C)   # vrwkv.py:184-186
    return _linear(y, P["output.weight"])


def channel_mix(x, P, patch_resolution, shift_pixel=1, gamma=0.25, eps=1e-5):
    """VRWKV_ChannelMix.forward (vrwkv.py:244-262); P: spatial_mix_k/r, key.weight (hidden, C), value.weight (C, hidden),
    receptance.weight and, with key_norm, key_norm.weight / key_norm.bias (hidden)."""
    from .qshift import q_shift_loops
    x = np.asarray(x, np.float64)
    B, T, C = x.shape
    xx = q_shift_loops(x, shift_pixel, gamma, patch_resolution) if shift_pixel > 0 else x
    xk, xr = (_mix(x, xx, P[n]) if shift_pixel > 0 else x for n in ("spatial_mix_k", "spatial_mix_r"))
    k = _linear(xk, P["key.weight"])
    has_norm = "key_norm.weight" in P
    k = row_epilogue(k, None, P["key_norm.weight"] if has_norm else None, P["key_norm.bias"] if has_norm else None,
                     None, PRE_RELU_SQ, POST_NONE, eps).reshape(B, T, -1)       # square(relu(k)), key_norm
    kv = _linear(k, P["value.weight"])
    return row_epilogue(kv, _linear(xr, P["receptance.weight"]), post=POST_SIGMOID_GATE).reshape(B, T, C)


def block(x, P, patch_resolution, wkv, layer_id, post_norm, shift_pixel=1, gamma=0.25, eps=1e-5):
    """Block.forward (vrwkv.py:296-313) without drop path.  P holds the block's parameters by the reference's names
    (ln0.* for layer 0, ln1.*, ln2.*, att.*, ffn.*, and gamma1 / gamma2 when the block has layer scale)."""
    x = np.asarray(x, np.float64)
    B, T, C = x.shape
    sub = lambda prefix: {n[len(prefix):]: a for n, a in P.items() if n.startswith(prefix)}
    ln = lambda a, n: row_epilogue(a, None, P[n + ".weight"], P[n + ".bias"], eps=eps).reshape(B, T, C)
    if layer_id == 0:
        x = ln(x, "ln0")
    for branch, norm, g in (("att", "ln1", "gamma1"), ("ffn", "ln2", "gamma2")):
        def run(inp):
            if branch == "att":
                return spatial_mix(inp, sub("att."), patch_resolution, wkv, shift_pixel, gamma, eps)
            return channel_mix(inp, sub("ffn."), patch_resolution, shift_pixel, gamma, eps)
        out = ln(run(x), norm) if post_norm else run(ln(x, norm))
        x = row_epilogue(out, x, None, None, P.get(g), PRE_NONE, POST_RESIDUAL).reshape(B, T, C)
    return x


def spatial_mix_v6(x, P, patch_resolution, wkv6, n_head, shift_pixel=1, with_cls_token=False, eps=1e-5):
    """VRWKV_SpatialMix_V6.forward (vrwkv6.py:175-228).  P: time_maa_x/w/k/v/r/g (C,), time_maa_w1 (C, 160),
    time_maa_w2 (5, 32, C), time_decay (C,), time_decay_w1 (C, 64), time_decay_w2 (64, C), time_faaaa (H, 64),
    key/value/receptance/gate/output .weight, ln_x.weight / ln_x.bias and, with key_norm, key_norm.*;
    wkv6(r, k, v, w, u, H) -> y is the operator to use (w: the raw decay logit, as RUN_CUDA_RWKV6 takes it)."""
    from .qshift import q_shift_multihead_loops
    x = np.asarray(x, np.float64)
    B, T, C = x.shape
    f = lambda n: np.asarray(P[n], np.float64)
    sx = q_shift_multihead_loops(x, shift_pixel, C // n_head, patch_resolution, with_cls_token)
    xx = sx - x                                                                   # :178-179
    xxx = x + xx * f("time_maa_x").reshape(-1)
    lo = np.tanh(xxx @ f("time_maa_w1")).reshape(B * T, 5, -1).transpose(1, 0, 2)  # (5, B*T, 32), :181-182
    m = np.einsum("fnd,fdc->fnc", lo, f("time_maa_w2")).reshape(5, B, T, C)       # :184-186
    xw, xk, xv, xr, xg = maa_mix(x, sx, m, [f("time_maa_" + n) for n in "wkvrg"])  # :188-192
    r, k, v = _linear(xr, P["receptance.weight"]), _linear(xk, P["key.weight"]), _linear(xv, P["value.weight"])
    gate = _linear(xg, P["gate.weight"])                                          # silu applied by groupnorm_gate, :197
    w = f("time_decay").reshape(-1) + np.tanh(xw @ f("time_decay_w1")) @ f("time_decay_w2")   # :199-201
    y = np.asarray(wkv6(r, k, v, w, f("time_faaaa"), n_head), np.float64)         # :217
    if "key_norm.weight" in P:
        y = row_epilogue(y, None, P["key_norm.weight"], P["key_norm.bias"], eps=eps).reshape(B, T, C)
    y = groupnorm_gate(y, gate, P["ln_x.weight"], P["ln_x.bias"], n_head, eps).reshape(B, T, C)   # :205-211
    return _linear(y, P["output.weight"])


def block_v6(x, P, patch_resolution, wkv6, n_head, layer_id, post_norm, shift_pixel=1, with_cls_token=False, eps=1e-5):
    """Block.forward of vrwkv6.py:314-332 without drop path; parameters by the reference's names as in `block`."""
    from .qshift import q_shift_multihead_loops
    x = np.asarray(x, np.float64)
    B, T, C = x.shape
    sub = lambda prefix: {n[len(prefix):]: a for n, a in P.items() if n.startswith(prefix)}
    ln = lambda a, n: row_epilogue(a, None, P[n + ".weight"], P[n + ".bias"], eps=eps).reshape(B, T, C)

    def ffn(inp):                                                                 # vrwkv6.py:271-286
        Pf = sub("ffn.")
        xx = q_shift_multihead_loops(inp, shift_pixel, C // n_head, patch_resolution, with_cls_token)
        k = _linear(_mix(inp, xx, Pf["spatial_mix_k"]), Pf["key.weight"])
        has_norm = "key_norm.weight" in Pf
        k = row_epilogue(k, None, Pf["key_norm.weight"] if has_norm else None, Pf["key_norm.bias"] if has_norm else None,
                         None, PRE_RELU_SQ, POST_NONE, eps).reshape(B, T, -1)
        return row_epilogue(_linear(k, Pf["value.weight"]), _linear(_mix(inp, xx, Pf["spatial_mix_r"]), Pf["receptance.weight"]),
                            post=POST_SIGMOID_GATE).reshape(B, T, C)

    att = lambda inp: spatial_mix_v6(inp, sub("att."), patch_resolution, wkv6, n_head, shift_pixel, with_cls_token, eps)
    if layer_id == 0:
        x = ln(x, "ln0")
    for run, norm, g in ((att, "ln1", "gamma1"), (ffn, "ln2", "gamma2")):
        out = ln(run(x), norm) if post_norm else run(ln(x, norm))
        x = row_epilogue(out, x, None, None, P.get(g), PRE_NONE, POST_RESIDUAL).reshape(B, T, C)
    return x
