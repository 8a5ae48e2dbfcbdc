"""Writes the golden fixtures of this directory from the CPU oracle (run from the repository root:
`python tests/golden/make_golden.py`).  The reference ships no vectors for this path, so these
fixtures freeze the oracle's answers on small seeded inputs: routing tables with many exact
ties, the cfg2 bucket offsets, and a few AdamW steps."""
import json
import math
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import bucket as OB  # noqa: E402
from oracle import moe as O  # noqa: E402
from piper_amd.configs import ADAMW, bucket_manifest_cfg2  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    g = torch.Generator().manual_seed(1234)
    T, E, K = 96, 16, 4
    logits = torch.round(torch.randn(T, E, generator=g) * 2.0) / 2.0   # coarse grid: many ties
    logits[0] = 0.0
    logits[1, 3] = -0.0
    scores, idx = O.route_topk(logits, K, route_norm=True)
    counts, starts, perm, inv = O.sort_by_expert(idx, E)
    np.savez(os.path.join(HERE, "routing_small.npz"), logits=logits.numpy(), top_k=np.int64(K),
             top_scores=scores.numpy(), top_idx=idx.numpy().astype(np.int32), counts=counts.numpy().astype(np.int32),
             starts=starts.numpy().astype(np.int32), perm=perm.numpy().astype(np.int32), inv_perm=inv.numpy().astype(np.int32))

    manifest = bucket_manifest_cfg2()
    numels = [math.prod(s) for _, s in manifest]
    offs, total = OB.plan_offsets(numels, 2, 256)
    with open(os.path.join(HERE, "bucket_offsets_cfg2.json"), "w") as f:
        json.dump({"elem_size": 2, "align_bytes": 256, "names": [n for n, _ in manifest], "numels": numels,
                   "offsets": offs, "total": total}, f)

    n = 1003
    p = torch.randn(n, generator=g) * 0.02
    m = torch.zeros(n)
    v = torch.zeros(n)
    grads, ps = [], [p.clone()]
    for step in range(1, 4):
        gr = torch.randn(n, generator=g) * 1e-3
        p, m, v = OB.adamw_step_torch(p, gr, m, v, step, ADAMW["lr"], ADAMW["betas"], ADAMW["eps"], ADAMW["weight_decay"])
        grads.append(gr)
        ps.append(p.clone())
    np.savez(os.path.join(HERE, "adamw_small.npz"), grads=torch.stack(grads).numpy(), params=torch.stack(ps).numpy(),
             exp_avg=m.numpy(), exp_avg_sq=v.numpy())
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
