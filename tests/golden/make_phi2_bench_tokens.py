#!/usr/bin/env python3
"""Writes tests/golden/phi2_bench_first_tokens.json: the first greedy tokens of the benchmark workload (full
Phi-2 architecture, bf16, the benchmark's seeded weights and 512-token prompt) as the CPU oracle computes them,
with the oracle's top-2 logit gap and largest logit magnitude at every step, so that a device token that differs
can be told from a near tie.  CPU only (about 12 GB of host memory, a few minutes on 8 cores):

    python tests/golden/make_phi2_bench_tokens.py [n_tokens]
"""
import json
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import phi2  # noqa: E402
from rai_amd import synthetic  # noqa: E402
from tests.util import synthetic_params  # noqa: E402


def main():
    n = int(sys.argv[1]) if len(sys.argv) > 1 else 17
    cfg = phi2.Config()
    params = synthetic_params(phi2.param_shapes(cfg), "bf16", seed=0)
    model = phi2.Model(cfg, params, "bf16")
    prompt = synthetic.prompt(cfg.vocab_size, 1, 512, seed=1)
    toks, logits_all = phi2.greedy_decode(model, prompt, n)
    gaps, mags = [], []
    for row in logits_all:
        r = np.sort(row[0].astype(np.float64))
        gaps.append(float(r[-1] - r[-2]))
        mags.append(float(np.max(np.abs(r))))
    out = {"workload": "Phi-2 architecture 32L bf16, seeded N(0,0.02) weights (seed 0), prompt synthetic.prompt(51200, 1, 512, seed=1)",
           "tokens": [int(t) for t in toks[0]], "top2_gap": gaps, "max_abs_logit": mags}
    path = Path(__file__).with_name("phi2_bench_first_tokens.json")
    path.write_text(json.dumps(out, indent=1) + "\n")
    print(path, out["tokens"])


if __name__ == "__main__":
    main()
