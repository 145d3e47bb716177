"""Writes tests/golden/int_cases.npz: small integer-valued cases whose products
are exact in fp32 in any accumulation order (|entries| <= 4, K <= 64, so every
partial sum is an integer below 2^11).  Expected outputs come from int64 numpy
arithmetic only - no code of the library or of the oracle is involved - so the
file pins both.  Run from the repository root:

    python tests/golden/make_int_fixtures.py
"""
import os

import numpy as np

CASES = {
    # name: (L, M, N, K)
    "tiny": (1, 5, 7, 3),
    "ragged": (2, 70, 200, 24),
    "wide": (1, 33, 1300, 64),
    "tall": (1, 1300, 40, 17),
}


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    for name, (L, M, N, K) in CASES.items():
        A = rng.integers(-4, 5, size=(L, M, K), dtype=np.int64)
        B = rng.integers(-4, 5, size=(L, K, N), dtype=np.int64)
        C = np.einsum("lmk,lkn->lmn", A, B)
        out[name + "_A"] = A.astype(np.int8)
        out[name + "_B"] = B.astype(np.int8)
        out[name + "_C"] = C.astype(np.int32)
        for dim, axis in ((1, 1), (2, 2)):
            out["%s_min%d_val" % (name, dim)] = C.min(axis=axis).astype(np.int32)
            out["%s_min%d_idx" % (name, dim)] = C.argmin(axis=axis).astype(np.int32)  # first occurrence
            # 128 largest per row, descending; missing candidates are marked with the int32 minimum
            Cr = C if dim == 2 else C.transpose(0, 2, 1)
            srt = -np.sort(-Cr, axis=-1)[..., :128]
            pad = 128 - srt.shape[-1]
            if pad > 0:
                srt = np.concatenate(
                    [srt, np.full(srt.shape[:-1] + (pad,), np.iinfo(np.int32).min, np.int64)], -1)
            out["%s_top%d_val" % (name, dim)] = srt.astype(np.int32)
        # a causal element mask and the masked product
        mask = np.tril(np.ones((M, N), dtype=bool))
        out[name + "_mask"] = mask
        out[name + "_Cmasked"] = np.where(mask[None], C, 0).astype(np.int32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "int_cases.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
