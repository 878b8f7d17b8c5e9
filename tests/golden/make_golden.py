"""Writes tests/golden/lora_small.npz: a small seeded multi-LoRA case with the
expected results of the whole path in the closed form
``y0 + scale * (x @ A_p) @ B_p`` evaluated in float64 on the DENSE matrices.

The reference stores no vectors for this path, so this fixture is self-generated
from the closed form; the paged pool inside it is packed with the oracle's
restatement of the reference packer (itself pinned in tests/test_oracle.py).
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "tests")]

from lora_cases import make_case, make_segments  # noqa: E402
from oracle import lora_oracle as O  # noqa: E402


def main():
    ranks = [8, 16, 32, 8]
    start, lens, ids = make_segments(77, 6, 1, 12, len(ranks))
    T = int(lens.sum())
    c = make_case(77, 128, ranks, batch=T, dtype="f16", bins=np.repeat(ids, lens), n_pages=4 * sum(ranks) + 11)
    rng = np.random.default_rng(78)
    y0 = O.round_to(rng.standard_normal((4, T, 128)).astype(np.float32), "f16")
    delta64 = np.zeros((4, T, 32))
    y64 = np.zeros((4, T, 128))
    for p in range(4):
        for t in range(T):
            a = c.bins[t]
            d = c.x[t].astype(np.float64) @ c.A[a][p].astype(np.float64)
            delta64[p, t, : ranks[a]] = d
            y64[p, t] = y0[p, t] + float(c.scales[a]) * (d @ c.B[a][p].astype(np.float64))
    np.savez_compressed(os.path.join(HERE, "lora_small.npz"), key=c.key.astype(np.float16),
                        value=c.value.astype(np.float16), a_start=c.a_start, a_len=c.a_len, a_loc=c.a_loc,
                        scales=c.scales.astype(np.float16), bins=c.bins, x=c.x.astype(np.float16),
                        y0=y0.astype(np.float16), delta64=delta64, y64=y64, ranks=np.array(ranks),
                        b_start_loc=start, b_seq_len=lens, b_indicies=ids)
    print("wrote lora_small.npz:", T, "tokens")


if __name__ == "__main__":
    main()
