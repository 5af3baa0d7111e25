"""What a literal run of the reference's CUDA kernel would return, as far as its 32-way token split goes
(oracle/chunk_carry.py): with the chunk-start carries multiplied by e^w the scheme IS the operator's formula; as
written it sits up to 1e-3 (T=196) away from it, less for longer sequences, and for T <= 32 (one token per lane) it
evaluates the other decay convention, |t-i| instead of |t-i|-1, exactly."""
import numpy as np

from oracle import biwkv, chunk_carry


def baseline_wu(C, T):
    c = np.arange(C)
    return (-5.0 + 8.0 * c / (C - 1)) / T, (np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T


def _closed(w, u, k, v, offset):
    """O(T^2) evaluation with decay exponent |t-i| - offset (offset 1 = the operator's formula)."""
    T = k.shape[0]
    t = np.arange(T)
    dist = np.abs(t[:, None] - t[None, :]) - offset
    out = np.empty_like(k)
    for c in range(k.shape[1]):
        wt = np.exp(k[None, :, c] - w[c] * dist)
        wt[t, t] = np.exp(u[c] + k[:, c])
        out[:, c] = (wt * v[None, :, c]).sum(1) / wt.sum(1)
    return out


def test_with_the_carry_factor_the_scheme_is_the_formula():
    rng = np.random.default_rng(0)
    for T in (33, 64, 196, 577):
        C = 12
        w, u = baseline_wu(C, T)
        k, v = rng.standard_normal((T, C)), rng.standard_normal((T, C))
        y = chunk_carry.biwkv_chunk_carry(w, u, k, v, carry_fix=True)
        ref = biwkv.biwkv_closed(w, u, k[None], v[None])[0]
        assert np.abs(y - ref).max() <= 1e-13, T
        assert np.abs(_closed(w, u, k, v, 1) - ref).max() <= 1e-13


def test_as_written_the_scheme_deviates_from_the_formula():
    rng = np.random.default_rng(1)
    seen = {}
    for T in (196, 577, 4150):
        C = 16 if T < 1000 else 4
        w, u = baseline_wu(C, T)
        k, v = rng.standard_normal((T, C)), rng.standard_normal((T, C))
        y = chunk_carry.biwkv_chunk_carry(w, u, k, v, carry_fix=False)
        ref = biwkv.biwkv_closed(w, u, k[None], v[None])[0]
        seen[T] = np.abs(y - ref).max(axis=0)               # per channel
    # T=196: every channel is off by more than fp32 rounding, the worst by 1e-4 ... 2e-3 (largest |w| = 3/T)
    assert seen[196].min() > 1e-6 and 1e-4 < seen[196].max() < 2e-3
    # the deviation is of order |w| = O(1/T): it shrinks with the sequence length
    assert seen[577].max() < 3e-4 and seen[4150].max() < 2e-5
    assert seen[4150].max() < seen[577].max() < seen[196].max()


def test_one_token_per_lane_is_the_other_convention():
    rng = np.random.default_rng(2)
    for T in (8, 20, 32):
        C = 6
        w, u = baseline_wu(C, T)
        k, v = rng.standard_normal((T, C)), rng.standard_normal((T, C))
        y = chunk_carry.biwkv_chunk_carry(w, u, k, v, carry_fix=False)
        assert np.abs(y - _closed(w, u, k, v, 0)).max() <= 1e-13
        assert np.abs(y - _closed(w, u, k, v, 1)).max() > 1e-3
