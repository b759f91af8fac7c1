"""Pins the oracle's activation dequantizers (patch lines 2744-2753, 2771-2774: to_float of A4 / A4H).

No data file of the reference holds a dequantized activation row. The reference does hold a second statement of the
same computation: `fake_quant_groups` in src/hessian.rs:70-92 ("the runtime's grouped activation quantizer ...
dequantized in place"), which quantizes a row per group (zero point, integer multiple 1..255 of the token's unit) and
writes back (q - z) * m * u. It is restated here in numpy from the Rust text, operation by operation in fp32, and
compared with quantize_row_a -> dequantize_row_a of the oracle (the quantizer itself is pinned by the compiled
reference's known answers):

  * the integers must agree exactly: the codes, zero points and multipliers that the Rust statement computes are the
    ones the oracle's dequantizer must have read back from the block fields (nibble order, the +8 offset of the
    stored codes, which header bits hold z and m of which subgroup, the unit in d);
  * the values: the C line forms (q - z) * (m * u), the Rust line ((q - z) * m) * u; (q - z) * m is an exact small
    integer, so the two differ by the rounding of m * u only. The test therefore demands bit equality with the C
    association applied to the Rust statement's integers, and at most one unit in the last place against the Rust
    association.

A4H rows: to_float must undo the rotation that from_float applied, so rotating the dequantized row forward again has
to give back the dequantized codes of the rotated row (H H^T = I up to rounding); the rotation is pinned on its own.
"""
import numpy as np
import pytest

f32 = np.float32


def fake_quant_groups_rust(row, clip, g):
    """src/hessian.rs:72-92. Returns the row as the Rust code leaves it, and q - z, m, u for the C association."""
    row = np.asarray(row, dtype=f32)
    clip = f32(clip)
    chunks = row.reshape(-1, g)
    lo = (np.minimum(chunks.min(axis=1), f32(0)) * clip).astype(f32)
    hi = (np.maximum(chunks.max(axis=1), f32(0)) * clip).astype(f32)
    r = f32(np.max((hi - lo).astype(f32)))
    if r == 0:
        r = f32(2.0)
    u = f32(r / f32(f32(15.0) * f32(255.0)))
    m = np.clip(np.ceil(((hi - lo).astype(f32) * f32(255.0)).astype(f32) / r), f32(1), f32(255)).astype(f32)
    inv = (f32(1.0) / (m * u).astype(f32)).astype(f32)
    z = np.clip(np.rint((-lo * inv).astype(f32)), f32(0), f32(15)).astype(f32)
    q = np.clip(np.rint((chunks * inv[:, None]).astype(f32)) + z[:, None], f32(0), f32(15)).astype(f32)
    d = (q - z[:, None]).astype(f32)
    rust = ((d * m[:, None]).astype(f32) * u).astype(f32).reshape(-1)
    return rust, d, m, u


def rows(kind, k, seed):
    rng = np.random.default_rng(seed)
    if kind == "normal":
        return rng.standard_normal(k).astype(f32)
    if kind == "outlier":
        x = rng.standard_normal(k).astype(f32)
        x[rng.integers(0, k, size=max(1, k // 200))] *= f32(20)
        return x
    if kind == "relu2":
        return (np.maximum(rng.standard_normal(k), 0) ** 2).astype(f32)
    if kind == "groups":
        return (rng.uniform(-1, 1, size=k) * np.exp2((np.arange(k) // 64) % 7 - 3)).astype(f32)
    if kind == "negative":
        return (-np.abs(rng.standard_normal(k))).astype(f32)
    raise ValueError(kind)


KINDS = ["normal", "outlier", "relu2", "groups", "negative"]


def ulps(a, b):
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, np.int64(-(2 ** 31)) - ia, ia)
    ib = np.where(ib < 0, np.int64(-(2 ** 31)) - ib, ib)
    return np.abs(ia - ib)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("k", [256, 1536, 5120])
@pytest.mark.parametrize("g", [64, 128, 256])
@pytest.mark.parametrize("clip", [1.0, 0.85])
def test_activation_dequantizer_matches_the_rust_statement(oracle, kind, k, g, clip):
    for seed in range(2):
        x = rows(kind, k, 7 * k + 13 * g + seed)
        blocks = oracle.quantize_row_a(x, clip=clip, G=g)
        got = oracle.dequantize_row_a(blocks)
        rust, d, m, u = fake_quant_groups_rust(x, clip, g)
        c_assoc = (d * (m * u).astype(f32)[:, None]).astype(f32).reshape(-1)   # patch line 2751
        assert got.dtype == f32 and got.shape == (k,)
        assert np.array_equal(got.view(np.uint32), c_assoc.view(np.uint32)), (kind, k, g, clip, seed)
        assert ulps(got, rust).max() <= 1, (kind, k, g, clip, seed)


def test_zero_row_dequantizes_to_zero(oracle):
    blocks = oracle.quantize_row_a(np.zeros(512, dtype=f32), clip=1.0, G=64)
    assert not oracle.dequantize_row_a(blocks).any()


@pytest.mark.parametrize("k,n_rot", [(256, 256), (1536, 1536), (5120, 5120), (5120, 1280)])
def test_rotated_activation_rows_come_back_unrotated(oracle, k, n_rot):
    x = rows("outlier", k, k + n_rot)
    blocks = oracle.quantize_row_a4h(x, clip=0.9, n_rot=n_rot, G=64)
    back = oracle.dequantize_row_a(blocks, hadamard=True)
    # forward rotation of to_float's output = the dequantized codes of the rotated row
    again = back.copy()
    for off in range(0, k, n_rot):
        again[off:off + n_rot] = oracle.hadamard(again[off:off + n_rot])
    codes = oracle.dequantize_row_a(blocks, hadamard=False)
    scale = np.abs(codes).max()
    assert np.abs(again - codes).max() <= 1e-5 * scale
    # and the whole trip stays within the quantization error of the rotated row (half a step of the widest group
    # inside the clip would be u * 255 / 2; outside the clip there is no bound, so compare energies instead)
    assert np.linalg.norm(back - x) <= 0.5 * np.linalg.norm(x)
