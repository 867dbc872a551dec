"""One process of tests/test_gpu_jit_cache.py: a reduced config-4 graph (products
with epilogues, elementwise groups) recorded and replayed; prints what the
recording cost and a checksum of the results as one JSON line."""
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def main():
    from tenncor_amd import graph, configs
    graph.set_evaluator("replay")
    g = graph.Graph()
    targets, x, _, _ = configs.config4_lstm(g, seq=5, batch=64, nin=32, hid=64)
    rng = np.random.default_rng(3)
    xs = rng.uniform(-1, 1, 64 * 5 * 32).astype(np.float32)
    for _ in range(3):
        g.assign(x, xs)
        g.evaluate(targets)
    st = graph.evaluator_stats()
    out = {k: st[k] for k in ("recorded", "replayed", "launches", "record_ms", "jit_ms", "jit_compiled", "jit_from_disk")}
    out["values"] = [t.get().astype(np.float64).sum() for t in targets]
    out["bits"] = [int(np.bitwise_xor.reduce(t.get().view(np.uint32).astype(np.uint64))) for t in targets]
    g.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
