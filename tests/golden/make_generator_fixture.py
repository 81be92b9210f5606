"""Writes tests/golden/generator_fixture.json from the tile lists the reference holds.

The reference keeps the output of its tile generator (engine/gen_kernel.cpp) as one macro line
per configuration in engine/mma_any/aq_bmma_impl/aq_bmma_w{p}a{q}.h.  Four of those lists are
reproduced exactly by the generator at K_STAGE=4 (w2a8, w3a3, w5a5, w7a7); the other eight come
from an earlier generator variant and are not used.  This script reads those four headers as
text (nothing is imported or executed), extracts the integer tuples, and stores per list the
count, a SHA-256 over the sorted tuples and the first / last tuple -- data, not source.

Run from the repository root in a container where /root/reference is mounted:
    python tests/golden/make_generator_fixture.py
"""
import hashlib
import json
import os
import re

REF = os.environ.get("ABQ_REFERENCE", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "generator_fixture.json")
LISTS = {"w2a8": (8, 2), "w3a3": (3, 3), "w5a5": (5, 5), "w7a7": (7, 7)}
LINE = re.compile(r"AQ_DECL_FUN\(AqBMMA,\s*(\d+),\s*(\d+),\s*(true|false),\s*" + r",\s*".join([r"(\d+)"] * 10) + r"\)")


def digest(tuples):
    h = hashlib.sha256()
    for t in sorted(tuples):
        h.update((",".join(str(v) for v in t) + "\n").encode())
    return h.hexdigest()


def main():
    out = {"k_stage": 4, "lists": {}}
    for name, (q, p) in LISTS.items():
        path = os.path.join(REF, "engine/mma_any/aq_bmma_impl/aq_bmma_%s.h" % name)
        tuples = []
        for m in LINE.finditer(open(path).read()):
            g = m.groups()
            tuples.append((int(g[0]), int(g[1]), 1 if g[2] == "true" else 0) + tuple(int(v) for v in g[3:]))
        assert all(t[0] == q and t[1] == p for t in tuples)
        out["lists"][name] = {
            "x_bits": q, "w_bits": p, "signed": 1, "count": len(tuples), "sha256_sorted": digest(tuples),
            "first": list(tuples[0]), "last": list(tuples[-1]),
        }
    json.dump(out, open(OUT, "w"), indent=1)
    print(json.dumps({k: v["count"] for k, v in out["lists"].items()}))


if __name__ == "__main__":
    main()
