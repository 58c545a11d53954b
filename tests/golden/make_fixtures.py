"""Writes tests/golden/extract_small.json: one tiny, fully spelled-out case of the extraction path.

Nothing here uses the oracle or the HIP library: every expected value comes from a brute-force Python loop over the
definition (count keys, sort by (count, key) descending, take the first floor(n * pct), copy rows), so the file pins
both of them from outside.  The reference holds no vectors for this path (its tests are end-to-end runs on GPUs); the
definitions followed are freq_recorder.cc:275-281 (rank order), optimal_solver_class.cc:1878 (top floor(n * pct / 100)
ranks are cached), cache_context.cu:2473 (capacity) and cache_context.cu:214-231 (out[i, :] = src[key[i], :]).

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import json
import os
import random


def main():
    rnd = random.Random(20240607)
    n_item, row_bytes, pct = 64, 16, 0.25
    table = [[rnd.randrange(256) for _ in range(row_bytes)] for _ in range(n_item)]
    # hotness stream: a skewed walk over a shuffled id space, long enough that every count is small and ties occur
    ids = list(range(n_item))
    rnd.shuffle(ids)
    stream = [ids[min(int(rnd.expovariate(0.15)), n_item - 1)] for _ in range(400)]
    counts = [0] * n_item
    for k in stream:
        counts[k] += 1
    seen = [k for k in range(n_item) if counts[k] > 0]
    ranked = sorted(seen, key=lambda k: (counts[k], k), reverse=True)  # (count desc, key desc)
    ranked += [k for k in range(n_item) if counts[k] == 0]             # never-seen keys follow in ascending order
    n_cached = int(n_item * (pct * 100 / 100.0))
    cached = sorted(ranked[:n_cached])
    capacity = int(n_item * (pct + 0.001))
    keys = [stream[rnd.randrange(len(stream))] for _ in range(24)] + [rnd.randrange(n_item) for _ in range(8)]
    out = [table[k] for k in keys]
    n_local = sum(1 for k in keys if k in set(cached))
    fixture = {
        "n_item": n_item, "row_bytes": row_bytes, "cache_percentage": pct, "table": table, "record_stream": stream,
        "rank_keys_observed": [k for k in ranked if counts[k] > 0],
        "rank_counts_observed": [counts[k] for k in ranked if counts[k] > 0],
        "cached_keys": cached, "capacity_rows": capacity, "lookup_keys": keys, "expected_output": out,
        "expected_group_offset": [0, n_local, len(keys)],
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "extract_small.json")
    with open(path, "w") as f:
        json.dump(fixture, f, separators=(",", ":"))
        f.write("\n")
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
