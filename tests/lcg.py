"""The fixed generator the reference known answers were produced with (exact in fp32), and FNV-1a 64."""
import numpy as np

from oracle.rq_oracle import BLOCK_DTYPE


class LCG:
    def __init__(self, seed):
        self.s = np.uint32(seed)

    def words(self, n):
        """n successive states (the state after each step), vectorised: s_{i+1} = a s_i + c mod 2^32."""
        out = np.empty(n, dtype=np.uint32)
        s = int(self.s)
        a, c = 1664525, 1013904223
        for i in range(n):
            s = (s * a + c) & 0xFFFFFFFF
            out[i] = s
        self.s = np.uint32(s)
        return out

    def uf(self, n):
        w = self.words(n)
        return (((w >> np.uint32(8)).astype(np.float32) / np.float32(16777216.0)) - np.float32(0.5)) * np.float32(4.0)


def fnv64(data: bytes) -> str:
    h = 1469598103934665603
    for b in data:
        h = ((h ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return "%016x" % h


def signed_nibbles(words):
    """uint32 words -> int8 codes, element 8w+j from bits [4j+3:4j]."""
    w = np.asarray(words, dtype=np.uint32)
    sh = (np.arange(8, dtype=np.uint32) * 4)
    nib = ((w[..., None] >> sh) & np.uint32(0xF)).astype(np.int8)
    nib = np.where(nib >= 8, nib - 16, nib).astype(np.int8)
    return nib.reshape(*w.shape[:-1], -1)


def act_row(k):
    return LCG(k).uf(k)


def weight_row(k):
    """One legacy-format weight row (k/256 blocks): random code words, d = 0.02, sum = row code sum."""
    g = LCG(k + 1)
    nb = k // 256
    row = np.zeros(nb, dtype=BLOCK_DTYPE)
    row["qs"] = g.words(nb * 32).reshape(nb, 32)
    total = int(signed_nibbles(row["qs"].reshape(-1)).astype(np.int64).sum())
    row["d"] = np.float32(0.02)
    row["sum"] = total
    row["pad"][:, 0] = k
    row["pad"][:, 1] = 0
    return row
