"""Writes tests/golden/doc_lengths.json: the document lengths of the benchmark configurations.

Seeded so every run sees the same documents:
  c3: 8 documents uniform in [512, 4096] summing to 16384 (rejection sampling on the last one)
  c4: log-uniform in [16, 256] until 16384 tokens, last truncated
  c5: one 32768-token document, then log-uniform in [1024, 16384], last truncated to fill 65536
Run once:  python tests/golden/make_doc_lengths.py
"""
import json
import math
import os
import random


def c3(seed=1337 + 3):
    rng = random.Random(seed)
    while True:
        first = [rng.randint(512, 4096) for _ in range(7)]
        last = 16384 - sum(first)
        if 512 <= last <= 4096:
            return first + [last]


def loguniform_fill(rng, lo, hi, total, first=()):
    out = list(first)
    while sum(out) < total:
        out.append(int(round(math.exp(rng.uniform(math.log(lo), math.log(hi))))))
    out[-1] -= sum(out) - total
    if out[-1] == 0:
        out.pop()
    return out


def main():
    data = {
        "c3": c3(),
        "c4": loguniform_fill(random.Random(1337 + 4), 16, 256, 16384),
        "c5": loguniform_fill(random.Random(1337 + 5), 1024, 16384, 65536, first=(32768,)),
    }
    for k, v in data.items():
        assert all(x > 0 for x in v)
    assert sum(data["c3"]) == 16384 and sum(data["c4"]) == 16384 and sum(data["c5"]) == 65536
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "doc_lengths.json")
    with open(path, "w") as f:
        json.dump(data, f)
    for k, v in data.items():
        print(k, len(v), "docs, sum L^2 =", sum(x * x for x in v), "max", max(v))


if __name__ == "__main__":
    main()
