"""Writes tests/golden/reference_known_answers.json.

The values are the known answers the compiled C reference (ggml-quants.c + ggml-cpu/quants.c with the
ruquant patch applied) printed for a fixed LCG input; they were recorded when the reference was surveyed
and are transcribed here as data. Nothing from the reference is imported or executed by this script.

Generator (exact in fp32): S <- S * 1664525 + 1013904223 (uint32); uf = ((S >> 8) / 2^24 - 0.5) * 4.
Activation row of length k: S = k, x[i] = uf(). Weight row: S = k + 1, qs words = next(); d = 0.02,
sum = the row's signed code sum, pad = {k, 0}. Hash = FNV-1a 64 over little-endian bytes.
"""
import json
import os

HADAMARD = [
    # k, p, m, fnv64 of the k output floats, bits of outputs 0, 1, k-1
    (256, 1, 256, "4ad857440ca5b34c", "3f83019b", "3f8aef4a", "bfe00000"),
    (1536, 12, 128, "cf84aa6ab12a0ecb", "3fd8228d", "3f5947d4", "00000000"),
    (4096, 1, 4096, "350ca3ac17aba724", "bfde5bd3", "bf6938b0", "bf880000"),
    (5120, 20, 256, "a807f40cda22835a", "3ffbe3dc", "bf333258", "bf0f1bbd"),
    (6144, 12, 512, "3efbea517b52eb9d", "bffa90aa", "c03cfe73", "c0234ca0"),
    (17408, 68, 256, "1e4a2bbfd44a1e64", "bec59801", "3ff973e0", "be1b390a"),
]

QUANT = """
256 Q 1.00 b58301e6587c64a8 3a888af5 00027787 faf7f2ff bf876406
256 QH 1.00 5e6dc06033300c84 3add65ee 00028888 ffb5c6cc bf27921c
256 Q 0.90 e531447a48c5a334 3a75c6eb 00027787 faf7f2ff bf9e1a8f
256 QH 0.90 a35886516e74d611 3ac74223 00028888 ffb5c6cc bf11d50b
256 Q 0.85 52fbb30d43bb0a54 3a681f6d 00027787 faf7f2ff bf95b81c
256 QH 0.85 05970a50181d364c 3abc303e 00028888 ffb5c6cc bec7b709
1536 Q 1.00 a2ae32e625634922 3a8868a5 00028778 f9fdfafe 3fdb0575
1536 QH 1.00 6c7a41f051a15520 3aeeb9cd 00027a97 bac6c9e6 40ac4633
1536 Q 0.90 78def1d22bd6b146 3a758929 00028778 f9fdfafe 40197aa2
1536 QH 0.90 ab26b753eefde839 3ad6da6b 00027a97 bac6c9e6 40b35189
1536 Q 0.85 ff3a1a531fd7b800 3a67e518 00028778 f9fdfafe 40127021
1536 QH 0.85 976d780c9cbcfa47 3acaeabc 00027a97 bac6c9e6 409da00f
4096 Q 1.00 24a1d66a75e0729a 3a88f53e 00028878 f4fbf5f7 41624a7c
4096 QH 1.00 874552a5261f7c0a 3b011efd 00028688 aed1bdb8 c00d6d8b
4096 Q 0.90 279283963dc76d56 3a76863c 00028878 f4fbf5f7 415efab7
4096 QH 0.90 8ad0046bfc95b4e5 3ae86afa 00028688 aed1bdb8 bfc7f3b7
4096 Q 0.85 7314fe64519fb412 3a68d41d 00028878 f4fbf5f7 4165652f
4096 QH 0.85 06803afd428056a1 3adb817b 00028688 aed1bdb8 c0128ded
5120 Q 1.00 a90d5a7f92878b9b 3a88d6f4 00027887 eefff9f8 be01ff67
5120 QH 1.00 58a91a4efd267729 3b09aa25 00027877 b1b79ea7 c1a4b54d
5120 Q 0.90 a3b2fa57075793ae 3a764fb6 00027887 eefff9f8 bf370a46
5120 QH 0.90 9b1434a00c24a4fb 3af7cbdb 00027877 b1b79ea7 c19a4abb
5120 Q 0.85 45bb2f1d6c7b2d6c 3a68a09e 00027887 eefff9f8 bed91209
5120 QH 0.85 14bdd3f5a15eb0a1 3aea07a6 00027877 b1b79ea7 c19e1346
6144 Q 1.00 051bde378a6b684b 3a88f41b 00028887 f4f8ecf8 bfca6442
6144 QH 1.00 3b1d918a4b07a7cf 3b036dac 00029788 bca6a2e1 41350849
6144 Q 0.90 2d4bbfdb60efef81 3a768430 00028887 f4f8ecf8 bf8fb619
6144 QH 0.90 3ee99ef7097474a8 3aec9235 00029788 bca6a2e1 41402180
6144 Q 0.85 867adf6b192b4605 3a68d22e 00028887 f4f8ecf8 bf88b5a7
6144 QH 0.85 016cfc473d97c476 3adf6da5 00029788 bca6a2e1 41300741
17408 Q 1.00 a906e371c0bec469 3a88d095 00028888 eff2fcf8 c01339bc
17408 QH 1.00 9e32966b9c12096a 3aff22ad 00027978 ccaed6a7 c1163604
17408 Q 0.90 8cdf52d820376dab 3a76443e 00028888 eff2fcf8 c06ddbde
17408 QH 0.90 0702a269878c3e6c 3ae59f35 00027978 ccaed6a7 c16ae317
17408 Q 0.85 00780cb69c277d9d 3a6895cb 00028888 eff2fcf8 c0869e23
17408 QH 0.85 fd28064e369d7f3b 3ad8dd79 00027978 ccaed6a7 c17f073e
"""

ROW_CODE_SUMS = {256: -123, 1536: -669, 4096: -2521, 5120: -2034, 6144: -2660, 17408: -9004}

ZERO_ROW = {"k": 512, "clip": 1.0, "u": "3a09119a", "sum0": "00020000", "pad0": "01010101",
            "code_word": "88888888"}


def main():
    had = [dict(k=k, p=p, m=m, fnv64=h, h0=a, h1=b, hlast=c) for k, p, m, h, a, b, c in HADAMARD]
    quant = []
    for line in QUANT.strip().splitlines():
        k, kind, clip, fnv, u, sum0, pad0, y = line.split()
        quant.append(dict(k=int(k), hadamard=kind == "QH", clip=clip, fnv64=fnv, u=u, sum0=sum0, pad0=pad0,
                          y=y))
    out = dict(hadamard=had, quant=quant, row_code_sums={str(k): v for k, v in ROW_CODE_SUMS.items()},
               zero_row=ZERO_ROW)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_known_answers.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")


if __name__ == "__main__":
    main()
