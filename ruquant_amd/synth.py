"""Synthetic inputs of the benchmark configurations: weight tensors written directly as W4A4 / W4A4H blocks
(random int4 codes, per-row fp32 scale, legacy code-sum header) and fp32 activations of several shapes."""
import numpy as np

from .w4a4 import BLOCK_DTYPE, TYPE_W4A4H


def signed_code_sums(qs):
    """qs: [..., n_words] uint32 -> per-leading-index sum of the signed int4 codes."""
    total = np.zeros(qs.shape[:-1], dtype=np.int64)
    for j in range(8):
        nib = (qs >> np.uint32(4 * j)) & np.uint32(0xF)
        total += nib.sum(axis=-1, dtype=np.int64) - 16 * (nib >= 8).sum(axis=-1, dtype=np.int64)
    return total


def random_weight_blocks(N, K, seed, type_, clip=0.0, n_rot=None):
    """[N, K/256] blocks: codes uniform in 0..15, d = |N(0.02, 0.005)| per row, sum = the row's code sum
    (legacy header, weight multiplier 1), pad[0] = K (or the Hadamard length), pad[1] = clip bits (0 = unset)."""
    rng = np.random.default_rng(seed)
    nb = K // 256
    blocks = np.zeros((N, nb), dtype=BLOCK_DTYPE)
    blocks["qs"] = rng.integers(0, 2 ** 32, size=(N, nb, 32), dtype=np.uint32)
    scale = np.abs(rng.normal(0.02, 0.005, size=N)).astype(np.float32)
    blocks["d"] = scale[:, None]
    blocks["sum"] = signed_code_sums(blocks["qs"].reshape(N, -1)).astype(np.int32)[:, None]
    blocks["pad"][:, :, 0] = (n_rot or K) if type_ == TYPE_W4A4H else K
    blocks["pad"][:, :, 1] = np.float32(clip).view(np.int32)
    return blocks


def activations(kind, M, K, seed):
    rng = np.random.default_rng(seed)
    if kind == "normal":
        return rng.standard_normal((M, K)).astype(np.float32)
    if kind == "outlier_channels":  # N(0,1) with 0.5 % of the channels scaled x20 (same channels for every token)
        x = rng.standard_normal((M, K)).astype(np.float32)
        ch = rng.choice(K, size=max(1, round(K * 0.005)), replace=False)
        x[:, ch] *= np.float32(20.0)
        return x
    if kind == "student_t4":  # Student-t, nu = 4, scaled to unit variance (var = nu / (nu - 2) = 2)
        return (rng.standard_t(4, size=(M, K)) / np.sqrt(2.0)).astype(np.float32)
    if kind == "relu2":  # max(N(0,1), 0)^2: non-negative, heavy right tail
        return (np.maximum(rng.standard_normal((M, K)), 0.0) ** 2).astype(np.float32)
    raise ValueError(kind)
