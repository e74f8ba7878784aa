"""Writes tests/golden/product_vectors.npz: operand pairs and the results of the
reference's own compiled C functional models (oracle/_ref, built from the
reference tree by oracle/Makefile).  Run in the container that holds the
reference tree:  python tests/golden/make_product_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import cpu  # noqa: E402
from tests.util import LUT_FILES, product_domain  # noqa: E402

N = 6000
out = {}
for kind, m in LUT_FILES:
    if kind == "ACC":
        continue
    a, b = product_domain(m, seed=900 + m, reps=1)
    rng = np.random.default_rng(m)
    # keep every special/boundary case at the tail, sample the bulk
    tail = 3000
    sel = np.concatenate([rng.choice(a.size - tail, N - tail, replace=False), np.arange(a.size - tail, a.size)])
    a, b = a[sel], b[sel]
    res = cpu.ref_model_array(kind, m, a.view(np.float32), b.view(np.float32))
    out[f"{kind}_{m}_a"], out[f"{kind}_{m}_b"], out[f"{kind}_{m}_out"] = a, b, res.view(np.uint32)
np.savez_compressed(os.path.join(ROOT, "tests", "golden", "product_vectors.npz"), **out)
print("wrote", len(out) // 3, "models x", N, "cases")
