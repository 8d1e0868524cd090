"""Writes tests/golden/attention_small.json: a tiny key-length-masked attention case evaluated by a pure-Python
float64 loop (no torch ops in the evaluation), used to pin the CPU oracle.

    python tests/golden/make_attention_golden.py

Inputs are small dyadic rationals so that the JSON text reproduces them exactly.
"""

from __future__ import annotations

import json
import math
import random
from pathlib import Path


def brute_force_attention(q, k, v, key_lengths, is_causal, zero_padded_queries):
    batch, heads, tq, d = len(q), len(q[0]), len(q[0][0]), len(q[0][0][0])
    tk = len(k[0][0])
    out = [[[[0.0] * d for _ in range(tq)] for _ in range(heads)] for _ in range(batch)]
    for b in range(batch):
        for h in range(heads):
            for i in range(tq):
                if zero_padded_queries and i >= key_lengths[b]:
                    continue
                visible = [j for j in range(tk) if j < key_lengths[b] and (not is_causal or j <= i)]
                if not visible:
                    continue
                scores = [sum(q[b][h][i][c] * k[b][h][j][c] for c in range(d)) / math.sqrt(d) for j in visible]
                top = max(scores)
                weights = [math.exp(s - top) for s in scores]
                total = sum(weights)
                for c in range(d):
                    out[b][h][i][c] = sum(w * v[b][h][j][c] for w, j in zip(weights, visible)) / total
    return out


def main() -> None:
    rng = random.Random(2026)
    batch, heads, tq, tk, d = 3, 2, 6, 6, 8

    def tensor(t):
        return [[[[rng.randint(-16, 16) / 8.0 for _ in range(d)] for _ in range(t)] for _ in range(heads)] for _ in range(batch)]

    q, k, v = tensor(tq), tensor(tk), tensor(tk)
    key_lengths = [6, 3, 0]
    cases = {}
    for name, causal, zero in (("plain", False, False), ("zero_padded", False, True), ("causal", True, False)):
        cases[name] = brute_force_attention(q, k, v, key_lengths, causal, zero)
    payload = {"q": q, "k": k, "v": v, "key_lengths": key_lengths, "expected": cases}
    path = Path(__file__).resolve().parent / "attention_small.json"
    path.write_text(json.dumps(payload))
    print("wrote", path)


if __name__ == "__main__":
    main()
