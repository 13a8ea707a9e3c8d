"""Writes tests/golden/generator_streams.json: FNV-1a 64 hashes and first bytes
of the seeded input streams (oracle_fill_random), so that this container and
the GPU box agree on every test input.  Uses only oracle/; the reference tree
holds no vectors for seeded data (its tests use constant patterns)."""
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
import __graft_entry__ as entry  # noqa: E402


def main():
    ora = entry.load_oracle()
    out = {"generator": "splitmix64-seeded xoshiro256**, little-endian bytes", "streams": []}
    for cfg in range(1, 6):
        seed = 0xB1170000 + cfg
        for n in (1, 64, 4099, 1 << 20):
            a = np.empty(n, dtype=np.uint8)
            ora.oracle_fill_random(a.ctypes.data, n, seed)
            out["streams"].append({
                "seed": "%x" % seed, "bytes": n,
                "fnv1a64": "%016x" % ora.oracle_fnv1a64(a.ctypes.data, n),
                "first8": a[:8].tolist(),
            })
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "generator_streams.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
