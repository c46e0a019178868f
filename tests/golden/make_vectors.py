"""Writes tests/golden/oracle_vectors.json: digests of what the CPU oracle produces on small seeded
cases.  The reference holds no golden vectors for this path, so these are NOT reference outputs:
they freeze the oracle (which is pinned by closed forms and library routines in tests/test_oracle.py)
so that a later edit that changes its results shows up as a failing test.

Run from the repository root:  python tests/golden/make_vectors.py"""
import hashlib
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from oracle import cq_oracle as O          # noqa: E402
from tests.util import make_case           # noqa: E402

CASES = [
    # name, (B, Hq, Hkv, D, T, R), bits, dtype, S
    ("cpu_reference_config", (1, 32, 8, 128, 1024, 0), 1, "fp16", 0),
    ("internvl_small_batch", (2, 32, 8, 128, 512, 70), 1, "bf16", 41),
    ("two_bit", (1, 16, 8, 128, 300, 33), 2, "bf16", 5),
]


def digest(a) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def vectors():
    out = {}
    for name, (B, Hq, Hkv, D, T, R), bits, dtype, S in CASES:
        c = make_case(B, Hq, Hkv, D, T, R, bits, dtype, seed=2024)
        kr = c["kr"] if R else None
        vr = c["vr"] if R else None
        o = O.decode_attention(c["q"], c["ck"], c["cv"], c["sk"], c["zk"], c["sv"], c["zv"], kr, vr, S, bits)
        out[name] = {
            "codes_k": digest(c["ck"]), "codes_v": digest(c["cv"]),
            "k_scale": digest(c["sk"].astype(np.float32)), "k_zero": digest(c["zk"].astype(np.float32)),
            "v_scale": digest(c["sv"].astype(np.float32)), "v_zero": digest(c["zv"].astype(np.float32)),
            # the attention output is floating point: kept as rounded values, compared with a tolerance
            "out_head0": [round(float(x), 6) for x in o[0, 0, :8]],
            "out_sum": round(float(np.asarray(o, dtype=np.float64).sum()), 4),
        }
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_vectors.json")
    with open(path, "w") as f:
        json.dump(vectors(), f, indent=1, sort_keys=True)
    print("wrote", path)
