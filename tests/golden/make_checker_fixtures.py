"""Writes tests/golden/checker_fixtures.npz from the reference's no-NPU checker compiled in place (oracle/_ref).

Run in a checkout that has the reference sources next to it:  python tests/golden/make_checker_fixtures.py
The fixtures are data only: the checker's default expert ids, its per-rank output blobs for ep_dispatch
([R*bs*K*h payload | bs*K assist tuples | R int32 recv counts | localE int64 token counts], reference:
tools/checker/src/oracle.cpp:661-708) and ep_combine ([bs, K, h] restored rows, reference:
tools/checker/src/executor.cpp:471-541).  Small cases are stored whole; the 4-rank 128x1024 case is stored as
SHA-256 digests of each rank's blob plus the event counts the reference CLI reports.
"""
import hashlib
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from oracle import ref  # noqa: E402

SMALL = [(2, 3, 4, 2, 4, 3), (4, 8, 16, 2, 8, 11), (4, 6, 64, 4, 16, 3)]
LARGE = [(4, 128, 1024, 2, 16, 11)]


def main():
    if not ref.available():
        raise SystemExit("oracle/_ref is not built (make -C oracle ref needs the reference sources)")
    out = {}
    for i, (R, bs, h, K, E, dtype) in enumerate(SMALL + LARGE):
        tag = f"case{i}"
        out[f"{tag}_shape"] = np.array([R, bs, h, K, E, dtype], np.int64)
        out[f"{tag}_ids"] = ref.checker_default_ids(R, bs, K, E)
        for op, name in ((0, "dispatch"), (1, "combine")):
            st, blobs, events = ref.checker_run(op, R, bs, h, K, E, dtype)
            assert st == 0
            out[f"{tag}_{name}_events"] = np.array([events], np.int64)
            if (R, bs, h, K, E, dtype) in SMALL:
                out[f"{tag}_{name}_blobs"] = np.stack([np.asarray(b, np.uint8) for b in blobs])
            else:
                digests = [hashlib.sha256(np.asarray(b, np.uint8).tobytes()).digest() for b in blobs]
                out[f"{tag}_{name}_sha256"] = np.frombuffer(b"".join(digests), np.uint8).reshape(R, 32)
    out["num_cases"] = np.array([len(SMALL) + len(LARGE)], np.int64)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "checker_fixtures.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
