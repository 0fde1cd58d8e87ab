"""Writes the fixtures in this directory.  Run from the repository root:

    python tests/golden/make_fixtures.py

reference_kats.json - the inline known-answer vectors of the reference's own tests
    (tests/unit/test_compress.py:292-419), transcribed as data: indices to pack, expected
    packed length, and, where the test's arithmetic fixes them, the packed bytes; the four
    _get_smaller_split answers.
codec_small.npz - one seeded 128x192 Student-t tensor with the oracle's coefficients,
    top-32 payload and reconstruction, so that a change of the oracle is noticed and the
    GPU tests have a committed input/output pair that does not depend on any RNG.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import codec as orc  # noqa: E402


def main():
    kats = {
        "pack_roundtrip": [
            {"name": "basic_0_to_5", "indices": [0, 1, 2, 3, 4, 5], "packed_len": 9,
             "packed": [0, 16, 0, 2, 48, 0, 4, 80, 0]},
            {"name": "two_rows", "indices": [10, 20, 30, 40, 50, 60, 70, 80], "packed_len": 12},
            {"name": "max_value", "indices": [4095, 4094, 0, 1], "packed_len": 6,
             "packed": [255, 239, 255, 0, 16, 0]},
            {"name": "beyond_8_bit", "indices": [0, 255, 256, 1000, 2000, 4000], "packed_len": 9},
            {"name": "arange_1000", "indices": list(range(1000)), "packed_len": 1500},
            {"name": "empty", "indices": [], "packed_len": 0},
        ],
        "smaller_split": [[64, 8, 8], [64, 7, 4], [64, 100, 64], [100, 16, 10]],
    }
    with open(os.path.join(HERE, "reference_kats.json"), "w") as fh:
        json.dump(kats, fh, indent=1)

    rng = np.random.default_rng(20240601)
    z = rng.standard_normal((4, 128, 192))
    x = (z[0] / np.sqrt((z[1] ** 2 + z[2] ** 2 + z[3] ** 2) / 3.0) * 1e-3).astype(np.float32)
    coef = orc.encode2d(x)
    idx12, val, xshape, totalk = orc.compress(coef, 32)
    recon = orc.decode2d(orc.decompress(idx12, val, xshape, totalk))
    np.savez_compressed(os.path.join(HERE, "codec_small.npz"), x=x, coef=coef, idx12=idx12, val=val, recon=recon)


if __name__ == "__main__":
    main()
