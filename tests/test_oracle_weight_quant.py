"""Pins the oracle's weight-side quantizer and dequantizers (patch lines 2507-2580, 2701-2710, 2738-2773).

No data file of the reference covers them, so the pins are:
  * the reference's own second statement of the row scale search and the code rule, `int4_scale` and `code` in
    src/gptq.rs:13-38 ("Matches quantize_row_w4a4_ref in our ggml"), restated here in numpy from the Rust text and
    compared bit for bit with the oracle's restatement of the C text;
  * the minimum property itself, in exact rational arithmetic: the chosen ratio has the smallest true squared error
    of the thirteen candidates (whenever the runner-up is not within rounding of it);
  * what the reference's tests assert about weight groups (src/gptq.rs:303-311: multipliers 1..15 with a 15 among
    them, header 1<<30 | k, unit in d) and the closed forms of the group lines (unit = largest scale / 15);
  * round trips: |dequantize(quantize(x)) - x| <= s / 2 inside the clip, and for W4A4H that rotating the
    dequantized row forward gives back code * scale (so to_float undoes exactly the rotation from_float applied).
"""
from fractions import Fraction

import numpy as np
import pytest

f32 = np.float32


def int4_scale_rust(row):
    """src/gptq.rs:13-34, operation by operation: f32 arithmetic, the error as a sequential f64 sum."""
    row = np.asarray(row, dtype=f32)
    amax = f32(np.max(np.abs(row))) if row.size else f32(0)
    if amax == 0:
        return f32(0)
    best_s, best_err = f32(0), np.inf
    for r in range(13):
        s = f32(f32(amax * f32(f32(1.0) - f32(f32(0.025) * f32(r)))) / f32(7.0))
        q = np.clip(np.rint(row / s), f32(-8), f32(7)).astype(f32)
        e = (q * s).astype(f32).astype(np.float64) - row.astype(np.float64)
        err = np.cumsum(e * e)[-1]          # cumsum adds left to right, as the iterator's sum does
        if err < best_err:
            best_err, best_s = err, s
    return best_s


def code_rust(row, s):
    """src/gptq.rs:36-38."""
    if s == 0:
        return np.zeros(len(row), dtype=np.int8)
    return np.clip(np.rint(np.asarray(row, dtype=f32) / f32(s)), -8, 7).astype(np.int8)


def signed_codes(blocks):
    words = blocks["qs"].reshape(-1)
    nib = (words[:, None] >> (4 * np.arange(8, dtype=np.uint32))[None, :]) & 0xF
    return (nib.astype(np.int16) - 16 * (nib >= 8)).reshape(-1).astype(np.int8)


def rows(kind, k, seed):
    rng = np.random.default_rng(seed)
    if kind == "normal":
        return rng.standard_normal(k).astype(f32)
    if kind == "heavy":
        return (rng.standard_t(3, size=k) * 0.02).astype(f32)
    if kind == "outlier":
        x = rng.standard_normal(k).astype(f32) * f32(0.01)
        x[rng.integers(k)] = 3.0
        return x
    if kind == "groups":
        return (rng.uniform(-1, 1, size=k) * np.exp2((np.arange(k) // 64) % 5 - 2)).astype(f32)
    if kind == "flat":
        return np.where(rng.uniform(size=k) < 0.5, -1.0, 1.0).astype(f32)
    raise ValueError(kind)


KINDS = ["normal", "heavy", "outlier", "groups", "flat"]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("k", [256, 1536, 5120])
def test_row_scale_and_codes_match_the_rust_statement(oracle, kind, k):
    for seed in range(3):
        x = rows(kind, k, 100 * k + seed)
        b = oracle.quantize_rows_w(x[None, :])[0]
        s = int4_scale_rust(x)
        assert b["d"][0].view(np.uint32) == s.view(np.uint32), (kind, k, seed, float(b["d"][0]), float(s))
        assert (b["d"] == b["d"][0]).all() and (b["pad"][:, 0] == k).all() and (b["pad"][:, 1] == 0).all()
        c = code_rust(x, s)
        assert (signed_codes(b) == c).all()
        assert (b["sum"] == int(c.astype(np.int64).sum())).all()      # legacy header: the row's code sum


def test_zero_row(oracle):
    b = oracle.quantize_rows_w(np.zeros((1, 512), dtype=f32))[0]
    assert (b["d"] == 0).all() and (b["sum"] == 0).all() and (b["qs"] == 0).all()
    assert (oracle.dequantize_row_w(b) == 0).all()


@pytest.mark.parametrize("kind", ["normal", "heavy", "outlier"])
def test_chosen_ratio_minimises_the_exact_error(oracle, kind):
    k = 256
    for seed in range(4):
        x = rows(kind, k, 7 + seed)
        b = oracle.quantize_rows_w(x[None, :])[0]
        amax = f32(np.max(np.abs(x)))
        cands = [f32(f32(amax * f32(f32(1.0) - f32(f32(0.025) * f32(r)))) / f32(7.0)) for r in range(13)]
        errs = []
        for s in cands:
            q = np.clip(np.rint(x / s), -8, 7).astype(f32)
            qs = (q * s).astype(f32)
            errs.append(sum((Fraction(float(a)) - Fraction(float(v))) ** 2 for a, v in zip(qs, x)))
        best = min(errs)
        order = sorted(errs)
        chosen = [i for i, s in enumerate(cands) if s.view(np.uint32) == b["d"][0].view(np.uint32)]
        assert chosen, "the stored scale is not one of the thirteen candidates"
        if order[1] - order[0] > best * Fraction(1, 10 ** 9):     # a clear winner: it must be the one stored
            assert errs[chosen[0]] == best


@pytest.mark.parametrize("wgroup,gs", [(256, 256), (64, 64)])
def test_weight_groups_structure(oracle, wgroup, gs):
    k = 2048
    x = rows("groups", k, 11)
    b = oracle.quantize_rows_w(x[None, :], wgroup=wgroup)[0]
    scales = np.array([int4_scale_rust(x[g * gs:(g + 1) * gs]) for g in range(k // gs)], dtype=f32)
    unit = f32(scales.max() / f32(15.0))
    assert (b["d"].view(np.uint32) == unit.view(np.uint32)).all()
    mult = np.clip(np.rint(scales / unit), 1, 15).astype(np.int32)
    assert mult.min() >= 1 and mult.max() == 15                    # src/gptq.rs:303
    for blk in range(k // 256):
        h = int(b["sum"][blk]) & 0xFFFFFFFF
        if gs == 256:
            assert h == (1 << 30 | int(mult[blk]))                 # src/gptq.rs:308
        else:
            m4 = mult[4 * blk:4 * blk + 4]
            assert h == (3 << 29 | int(m4[0]) | int(m4[1]) << 4 | int(m4[2]) << 8 | int(m4[3]) << 12)
    want = np.concatenate([code_rust(x[g * gs:(g + 1) * gs], f32(f32(mult[g]) * unit)) for g in range(k // gs)])
    assert (signed_codes(b) == want).all()
    # the dequantizer reads the multipliers the same way (src/gptq.rs:313-319)
    deq = oracle.dequantize_row_w(b)
    per = np.repeat(mult, gs).astype(f32) * unit
    assert (deq.view(np.uint32) == (want.astype(f32) * per).astype(f32).view(np.uint32)).all()


@pytest.mark.parametrize("k", [512, 1536, 5120])
def test_round_trip_inside_the_clip(oracle, k):
    x = rows("normal", k, k)
    b = oracle.quantize_rows_w(x[None, :])[0]
    s = float(b["d"][0])
    deq = oracle.dequantize_row_w(b)
    inside = np.abs(x) <= 7.0 * s
    assert inside.sum() > k // 2
    assert (np.abs(deq[inside] - x[inside]) <= 0.5 * s * (1 + 1e-6)).all()


@pytest.mark.parametrize("k,n_rot", [(512, 512), (1536, 1536), (5120, 5120), (5120, 2560), (1536, 768)])
def test_rotated_weights_round_trip(oracle, k, n_rot):
    x = rows("normal", k, 3 * k + n_rot)
    b = oracle.quantize_rows_w(x[None, :], hadamard=True, n_rot=n_rot)[0]
    assert (b["pad"][:, 0] == n_rot).all()
    rot = np.concatenate([oracle.hadamard(x[o:o + n_rot]) for o in range(0, k, n_rot)])
    # the stored codes are those of the rotated row
    plain = oracle.quantize_rows_w(rot[None, :])[0]
    assert (b["qs"] == plain["qs"]).all() and (b["d"] == plain["d"]).all() and (b["sum"] == plain["sum"]).all()
    # to_float comes back to the original basis: rotating it forward again gives code * scale up to rounding
    deq = oracle.dequantize_row_w(b, hadamard=True)
    again = np.concatenate([oracle.hadamard(deq[o:o + n_rot]) for o in range(0, k, n_rot)])
    grid = signed_codes(b).astype(f32) * b["d"][0]
    assert np.abs(again - grid).max() <= 1e-5 * np.abs(grid).max()
    assert np.linalg.norm(deq - x) / np.linalg.norm(x) < 0.2
