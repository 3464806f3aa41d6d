"""Writes tests/golden/config1_oracle.npz: the oracle's results for config 1 of BASELINE.json (256 tokens, hidden 512,
8 experts top-2 softmax, intermediate 1024, seed 0).  The reference holds no vectors for this path and cannot run
here (JAX is absent), so these are the oracle's own values, frozen: integer results in full, the bf16 output as a
checksum plus a few rows.  They guard the oracle (and through it the GPU path) against silent change."""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import moe_oracle as O  # noqa: E402
from tests import helpers as H  # noqa: E402


def build():
    prob = H.make_problem(M=256, D=512, E=8, k=2, I=1024, seed=0)
    ref = O.moe_experts(prob["x"], prob["logits"], prob["experts"], top_k=2)
    bits = O.f32_to_bf16_bits(ref["out"])
    return dict(indices=ref["indices"], weights=ref["weights"], group_sizes=ref["group_sizes"],
                sorted_token_ids=ref["sorted_token_ids"], inv_perm=ref["inv_perm"],
                out_rows=np.array([0, 1, 100, 255]), out_bits=bits[[0, 1, 100, 255]],
                out_sha256=np.frombuffer(hashlib.sha256(bits.tobytes()).digest(), dtype=np.uint8),
                x_sha256=np.frombuffer(hashlib.sha256(prob["x"].tobytes()).digest(), dtype=np.uint8),
                gate_codes_sha256=np.frombuffer(hashlib.sha256(prob["experts"]["gate"][0].tobytes()).digest(), dtype=np.uint8))


if __name__ == "__main__":
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1_oracle.npz"), **build())
    print("written")
