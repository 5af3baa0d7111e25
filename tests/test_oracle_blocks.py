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


def _torch_block(x, P, res, layer_id, post_norm, key_norm, shift_pixel=1, gamma=0.25):
    """The block written a second time, with torch float64 tensor ops and the slice-copy shift of vrwkv.py:68-79, and
    the softmax form of the operator (y_t = sum_i W[t,i] v_i / sum_i W[t,i], W[t,i] = exp(k_i - w(|t-i|-1)), exp(u+k_t))."""
    tt = {n: torch.from_numpy(np.asarray(a, np.float64)) for n, a in P.items()}
    B, T, C = x.shape

    def shift(a):
        Hp, Wp = res
        Cc = a.shape[2]
        i = a.transpose(1, 2).reshape(B, Cc, Hp, Wp)
        o = torch.zeros_like(i)
        g1, g2, g3, g4 = (int(Cc * gamma * q) for q in (1, 2, 3, 4))
        s = shift_pixel
        o[:, 0:g1, :, s:Wp] = i[:, 0:g1, :, 0:Wp - s]
        o[:, g1:g2, :, 0:Wp - s] = i[:, g1:g2, :, s:Wp]
        o[:, g2:g3, s:Hp, :] = i[:, g2:g3, 0:Hp - s, :]
        o[:, g3:g4, 0:Hp - s, :] = i[:, g3:g4, s:Hp, :]
        o[:, g4:] = i[:, g4:]
        return o.flatten(2).transpose(1, 2)

    def wkv(w, u, k, v):
        idx = torch.arange(T)
        dist = (idx[:, None] - idx[None, :]).abs().double() - 1.0
        logw = k[:, None, :, :] - w[None, None, None, :] * dist[None, :, :, None]           # (B, t, i, C)
        eye = torch.eye(T, dtype=torch.bool)[None, :, :, None]
        logw = torch.where(eye, (u[None, None, :] + k)[:, None, :, :].expand(B, T, T, C), logw)
        return (torch.softmax(logw, dim=2) * v[:, None, :, :]).sum(2)

    def att(a):
        xx = shift(a)
        mk, mv, mr = (tt["att.spatial_mix_" + n].reshape(1, 1, -1) for n in "kvr")
        k = F.linear(a * mk + xx * (1 - mk), tt["att.key.weight"])
        v = F.linear(a * mv + xx * (1 - mv), tt["att.value.weight"])
        r = F.linear(a * mr + xx * (1 - mr), tt["att.receptance.weight"])
        y = wkv(tt["att.spatial_decay"] / T, tt["att.spatial_first"] / T, k, v)
        if key_norm:
            y = F.layer_norm(y, (C,), tt["att.key_norm.weight"], tt["att.key_norm.bias"], 1e-5)
        return F.linear(torch.sigmoid(r) * y, tt["att.output.weight"])

    def ffn(a):
        xx = shift(a)
        mk, mr = (tt["ffn.spatial_mix_" + n].reshape(1, 1, -1) for n in "kr")
        k = torch.square(torch.relu(F.linear(a * mk + xx * (1 - mk), tt["ffn.key.weight"])))
        if key_norm:
            k = F.layer_norm(k, (k.shape[-1],), tt["ffn.key_norm.weight"], tt["ffn.key_norm.bias"], 1e-5)
        return torch.sigmoid(F.linear(a * mr + xx * (1 - mr), tt["ffn.receptance.weight"])) * F.linear(k, tt["ffn.value.weight"])

    ln = lambda a, n: F.layer_norm(a, (C,), tt[n + ".weight"], tt[n + ".bias"], 1e-5)
    h = torch.from_numpy(np.asarray(x, np.float64))
    if layer_id == 0:
        h = ln(h, "ln0")
    for f, n, g in ((att, "ln1", "gamma1"), (ffn, "ln2", "gamma2")):
        out = ln(f(h), n) if post_norm else f(ln(h, n))
        h = h + (tt[g] * out if g in tt else out)
    return h.numpy()


def _block_params(rng, C, hidden, key_norm, layer_scale, layer_id):
    P = {}
    for n in ("ln1", "ln2") + (("ln0",) if layer_id == 0 else ()):
        P[n + ".weight"], P[n + ".bias"] = rng.uniform(0.5, 1.5, C), rng.normal(0, 0.2, C)
    for n in "kvr":
        P["att.spatial_mix_" + n] = rng.uniform(0, 1, C)
    for n in "kr":
        P["ffn.spatial_mix_" + n] = rng.uniform(0, 1, C)
    for n in ("key", "value", "receptance", "output"):
        P[f"att.{n}.weight"] = rng.normal(0, C ** -0.5, (C, C))
    P["att.spatial_decay"], P["att.spatial_first"] = rng.uniform(-5, 3, C), rng.uniform(-1, 1, C)
    P["ffn.key.weight"] = rng.normal(0, C ** -0.5, (hidden, C))
    P["ffn.value.weight"] = rng.normal(0, hidden ** -0.5, (C, hidden))
    P["ffn.receptance.weight"] = rng.normal(0, C ** -0.5, (C, C))
    if key_norm:
        P["att.key_norm.weight"], P["att.key_norm.bias"] = rng.uniform(0.5, 1.5, C), rng.normal(0, 0.2, C)
        P["ffn.key_norm.weight"], P["ffn.key_norm.bias"] = rng.uniform(0.5, 1.5, hidden), rng.normal(0, 0.2, hidden)
    if layer_scale:
        P["gamma1"], P["gamma2"] = rng.uniform(0.2, 1.0, C), rng.uniform(0.2, 1.0, C)
    return P


def test_block_composition_against_torch_ops_in_every_variant():
    """oracle.blocks.block (loops, row epilogues, q_shift loops, the operator oracle's recurrence) against the same
    block written with torch float64 ops, slice-copy shifts and the operator's softmax form: a swapped mix, a norm on
    the wrong side of the branch, a gate before the norm or a missing 1/T on the decays would each show."""
    from oracle import biwkv
    rng = np.random.default_rng(11)
    B, res, C, hidden = 2, (3, 4), 16, 40
    T = res[0] * res[1]
    wkv = lambda w, u, k, v: biwkv.biwkv_scan(np.asarray(w), np.asarray(u), np.asarray(k), np.asarray(v))
    for layer_id in (0, 1):
        for post_norm in (False, True):
            for key_norm in (False, True):
                for layer_scale in (False, True):
                    P = _block_params(rng, C, hidden, key_norm, layer_scale, layer_id)
                    x = rng.standard_normal((B, T, C))
                    got = blocks.block(x, P, res, wkv, layer_id, post_norm)
                    want = _torch_block(x, P, res, layer_id, post_norm, key_norm)
                    assert np.allclose(got, want, rtol=0, atol=1e-10), (layer_id, post_norm, key_norm, layer_scale)


def test_block_special_cases_by_hand():
    """Identity projections, mixes of one (no shifted share), constant decay zero: the spatial mix is sigmoid(x) times
    the plain mean-like weighting of x itself, and with u = 0, w = 0 every token weighs e^{k_i}: y_t = sum e^{x_i} x_i /
    sum e^{x_i} for all t."""
    from oracle import biwkv
    B, res, C = 1, (2, 2), 4
    T = 4
    rng = np.random.default_rng(5)
    x = rng.standard_normal((B, T, C))
    eye = np.eye(C)
    P = {"spatial_mix_k": np.ones(C), "spatial_mix_v": np.ones(C), "spatial_mix_r": np.ones(C), "key.weight": eye,
         "value.weight": eye, "receptance.weight": eye, "output.weight": eye, "spatial_decay": np.zeros(C),
         "spatial_first": np.zeros(C)}
    wkv = lambda w, u, k, v: biwkv.biwkv_scan(np.asarray(w), np.asarray(u), np.asarray(k), np.asarray(v))
    got = blocks.spatial_mix(x, P, res, wkv)
    # w = 0: decay^(|t-i|-1) = 1 for i != t, and e^{u + k_t} = e^{k_t} for i = t
    y = (np.exp(x) * x).sum(1, keepdims=True) / np.exp(x).sum(1, keepdims=True)
    want = y / (1.0 + np.exp(-x))
    assert np.allclose(got, want, rtol=0, atol=1e-12)
    # channel mix with identity key / value (hidden = C), no key_norm: sigmoid(x) * relu(x)^2
    Pf = {"spatial_mix_k": np.ones(C), "spatial_mix_r": np.ones(C), "key.weight": eye, "value.weight": eye,
          "receptance.weight": eye}
    assert np.allclose(blocks.channel_mix(x, Pf, res), np.maximum(x, 0) ** 2 / (1.0 + np.exp(-x)), rtol=0, atol=1e-12)


def _torch_block_v6(x, P, res, H, layer_id, post_norm, key_norm, with_cls):
    """The VRWKV6 block a second time: torch float64 ops as vrwkv6.py writes them, the slice-copy per-head shift of
    vrwkv6.py:75-100, and the operator as a plain token loop over a (H, 64, 64) state in both directions."""
    tt = {n: torch.from_numpy(np.asarray(a, np.float64)) for n, a in P.items()}
    B, T, C = x.shape
    hd = C // H

    def shift(a, s=1):
        cls = a[:, -1:, :] if with_cls else None
        body = a[:, :-1, :] if with_cls else a
        Hp, Wp = res
        i = body.transpose(1, 2).reshape(B, -1, hd, Hp, Wp)
        o = torch.zeros_like(i)
        q = hd // 4
        o[:, :, 0:q, :, s:Wp] = i[:, :, 0:q, :, 0:Wp - s]
        o[:, :, q:2 * q, :, 0:Wp - s] = i[:, :, q:2 * q, :, s:Wp]
        o[:, :, 2 * q:3 * q, s:Hp, :] = i[:, :, 2 * q:3 * q, 0:Hp - s, :]
        o[:, :, 3 * q:4 * q, 0:Hp - s, :] = i[:, :, 3 * q:4 * q, s:Hp, :]
        o = o.reshape(B, C, -1).transpose(1, 2)
        return torch.cat((o, cls), dim=1) if with_cls else o

    def wkv6(r, k, v, w, u):
        d = torch.exp(-torch.exp(w)).reshape(B, T, H, hd)
        r, k, v = (a.reshape(B, T, H, hd) for a in (r, k, v))
        y = torch.zeros(B, T, H, hd, dtype=torch.float64)
        for order, bonus in ((range(T), True), (range(T - 1, -1, -1), False)):
            S = torch.zeros(B, H, hd, hd, dtype=torch.float64)                      # S[j, i]
            for t in order:
                kv = k[:, t, :, :, None] * v[:, t, :, None, :]
                y[:, t] += torch.einsum("bhj,bhji->bhi", r[:, t], (u[None, :, :, None] * kv if bonus else 0) + S)
                S = d[:, t, :, :, None] * S + kv
        return y.reshape(B, T, C)

    def att(a):
        sx = shift(a)
        xx = sx - a
        xxx = a + xx * tt["att.time_maa_x"]
        lo = torch.tanh(xxx @ tt["att.time_maa_w1"]).view(B * T, 5, -1).transpose(0, 1)
        mw, mk, mv, mr, mg = torch.bmm(lo, tt["att.time_maa_w2"]).view(5, B, T, -1).unbind(0)
        xw, xk, xv, xr, xg = (a + xx * (tt["att.time_maa_" + n] + m) for n, m in zip("wkvrg", (mw, mk, mv, mr, mg)))
        r, k, v = F.linear(xr, tt["att.receptance.weight"]), F.linear(xk, tt["att.key.weight"]), F.linear(xv, tt["att.value.weight"])
        g = F.silu(F.linear(xg, tt["att.gate.weight"]))
        w = tt["att.time_decay"] + torch.tanh(xw @ tt["att.time_decay_w1"]) @ tt["att.time_decay_w2"]
        y = wkv6(r, k, v, w, tt["att.time_faaaa"])
        if key_norm:
            y = F.layer_norm(y, (C,), tt["att.key_norm.weight"], tt["att.key_norm.bias"], 1e-5)
        y = F.group_norm(y.reshape(B * T, C), H, tt["att.ln_x.weight"], tt["att.ln_x.bias"], 1e-5).view(B, T, C)
        return F.linear(y * g, tt["att.output.weight"])

    def ffn(a):
        xx = shift(a)
        mk, mr = tt["ffn.spatial_mix_k"], tt["ffn.spatial_mix_r"]
        k = torch.square(torch.relu(F.linear(a * mk + xx * (1 - mk), tt["ffn.key.weight"])))
        if key_norm:
            k = F.layer_norm(k, (k.shape[-1],), tt["ffn.key_norm.weight"], tt["ffn.key_norm.bias"], 1e-5)
        return torch.sigmoid(F.linear(a * mr + xx * (1 - mr), tt["ffn.receptance.weight"])) * F.linear(k, tt["ffn.value.weight"])

    ln = lambda a, n: F.layer_norm(a, (C,), tt[n + ".weight"], tt[n + ".bias"], 1e-5)
    h = torch.from_numpy(np.asarray(x, np.float64))
    if layer_id == 0:
        h = ln(h, "ln0")
    for f, n, g in ((att, "ln1", "gamma1"), (ffn, "ln2", "gamma2")):
        out = ln(f(h), n) if post_norm else f(ln(h, n))
        h = h + (tt[g] * out if g in tt else out)
    return h.numpy()


def test_vrwkv6_block_composition_against_torch_ops():
    """oracle.blocks.block_v6 (maa_mix, groupnorm_gate, row epilogues, the per-head shift loops and the operator
    oracle's recurrence) against the block written with torch float64 ops and a plain state loop for the operator:
    norm placement, layer scale, key_norm, a class token, and the order of the five mixes."""
    from oracle import wkv6 as o6
    rng = np.random.default_rng(23)
    B, res, H = 2, (2, 3), 2
    C, hidden = H * 64, 3 * H * 64
    wk = lambda r, k, v, w, u, Hh: o6.wkv6_scan(r, k, v, w, u, Hh)
    for layer_id, post_norm, key_norm, layer_scale, with_cls in ((0, True, False, True, False), (1, False, True, False, True),
                                                                 (1, True, True, True, True), (0, False, False, False, False)):
        T = res[0] * res[1] + (1 if with_cls else 0)
        P = {}
        for n in ("ln1", "ln2") + (("ln0",) if layer_id == 0 else ()):
            P[n + ".weight"], P[n + ".bias"] = rng.uniform(0.5, 1.5, C), rng.normal(0, 0.2, C)
        for n in "xwkvrg":
            P["att.time_maa_" + n] = rng.uniform(0, 1, C)
        P["att.time_maa_w1"], P["att.time_maa_w2"] = rng.normal(0, 0.1, (C, 160)), rng.normal(0, 0.1, (5, 32, C))
        P["att.time_decay"] = rng.uniform(-3, 0.5, C)
        P["att.time_decay_w1"], P["att.time_decay_w2"] = rng.normal(0, 0.1, (C, 64)), rng.normal(0, 0.1, (64, C))
        P["att.time_faaaa"] = rng.normal(0, 0.3, (H, 64))
        for n in ("key", "value", "receptance", "gate", "output"):
            P[f"att.{n}.weight"] = rng.normal(0, C ** -0.5, (C, C))
        P["att.ln_x.weight"], P["att.ln_x.bias"] = rng.uniform(0.5, 1.5, C), rng.normal(0, 0.2, C)
        P["ffn.spatial_mix_k"], P["ffn.spatial_mix_r"] = rng.uniform(0, 1, C), rng.uniform(0, 1, C)
        P["ffn.key.weight"] = rng.normal(0, C ** -0.5, (hidden, C))
        P["ffn.value.weight"] = rng.normal(0, hidden ** -0.5, (C, hidden))
        P["ffn.receptance.weight"] = rng.normal(0, C ** -0.5, (C, C))
        if key_norm:
            P["att.key_norm.weight"], P["att.key_norm.bias"] = rng.uniform(0.5, 1.5, C), rng.normal(0, 0.2, C)
            P["ffn.key_norm.weight"], P["ffn.key_norm.bias"] = rng.uniform(0.5, 1.5, hidden), rng.normal(0, 0.2, hidden)
        if layer_scale:
            P["gamma1"], P["gamma2"] = rng.uniform(0.2, 1.0, C), rng.uniform(0.2, 1.0, C)
        x = rng.standard_normal((B, T, C))
        got = blocks.block_v6(x, P, res, wk, H, layer_id, post_norm, with_cls_token=with_cls)
        want = _torch_block_v6(x, P, res, H, layer_id, post_norm, key_norm, with_cls)
        assert np.allclose(got, want, rtol=0, atol=1e-9), (layer_id, post_norm, key_norm, layer_scale, with_cls,
                                                            np.abs(got - want).max())
