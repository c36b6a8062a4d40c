"""Writes tests/golden/top2_gating_small.json and switch_gating_small.json from
the CPU oracle.

The reference holds no test, golden vector or fixture for its MoE file, and its
TensorFlow dependency is not installed, so these vectors come from the oracle
(whose functions are pinned independently in tests/test_oracle.py); they guard
the oracle and the HIP path against drifting together.

  python tests/golden/make_golden.py
"""

import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import moe_oracle as O  # noqa: E402


def main():
  rng = np.random.default_rng(20260101)
  g, s, e, c = 2, 24, 5, 6
  logits = np.round(rng.standard_normal((g, s, e)) * 8) / 8   # exact in float32
  logits = logits.astype(np.float32)
  r = O.top_2_gating(logits, c)
  out = dict(capacity=c, logits=logits.tolist(), loss=float(r["loss"]))
  for k in ("index_1", "index_2", "pos_1", "pos_2", "kept_1", "kept_2"):
    out[k] = r[k].astype(int).tolist()
  for k in ("gate_1", "gate_2"):
    out[k] = [[float(v) for v in row] for row in r[k]]
  with open(os.path.join(HERE, "top2_gating_small.json"), "w") as f:
    json.dump(out, f)

  # switch gating on the same logits, with a padding mask and the z-loss
  imp = (rng.random((g, s)) < 0.8).astype(np.float32)
  r = O.switch_gating(logits, c, importance=imp, train=True, z_loss=1e-2,
                      num_microbatches=2)
  out = dict(capacity=c, logits=logits.tolist(), importance=imp.tolist(),
             z_loss=1e-2, num_microbatches=2, loss=float(r["loss"]))
  for k in ("index_1", "pos_1", "kept_1"):
    out[k] = r[k].astype(int).tolist()
  out["gate_1"] = [[float(v) for v in row] for row in r["gate_1"]]
  with open(os.path.join(HERE, "switch_gating_small.json"), "w") as f:
    json.dump(out, f)


if __name__ == "__main__":
  main()
