"""Writes tests/golden/qk_rope_embedding_small.json: tiny cases of the query / key RMSNorm + rotary embedding and of
the embedding-bag mean, evaluated by pure-Python float64 loops (no torch, no numpy), used to pin the CPU oracle and as
committed expected outputs for the float32 GPU paths.

    python tests/golden/make_widened_golden.py

Inputs are small dyadic rationals so that the JSON text reproduces them exactly. The rules restated here:
- RMSNorm over the whole model width, then per head a rotation of the feature pairs (2i, 2i + 1) by the angle
  position * base ** (-2i / rotary_dim), rotary_dim = 2 * (head_dim // 2), an odd last feature left as it is
  (experiments/tokenformer/model.py:131-136, 149-154, 165-192; experiments/symbiosis/backbone.py:33-36);
- the mean over the non-zero ids of a bag, zeros for a bag of padding only
  (accelerators/embedding/embedding_bag.py:82-83).
"""

from __future__ import annotations

import json
import math
import random
from pathlib import Path


def dyadic(rng: random.Random, span: int = 16, denominator: int = 8) -> float:
    return rng.randint(-span, span) / denominator


def rms_norm_row(row, weight, eps):
    mean_square = sum(value * value for value in row) / len(row)
    scale = 1.0 / math.sqrt(mean_square + eps)
    return [value * scale * w for value, w in zip(row, weight)]


def rotate_row(row, position, num_heads, rope_base):
    head_dim = len(row) // num_heads
    rotary_dim = (head_dim // 2) * 2
    out = list(row)
    for head in range(num_heads):
        base = head * head_dim
        for pair in range(rotary_dim // 2):
            angle = position * rope_base ** (-(2 * pair) / max(1, rotary_dim))
            even, odd = row[base + 2 * pair], row[base + 2 * pair + 1]
            out[base + 2 * pair] = even * math.cos(angle) - odd * math.sin(angle)
            out[base + 2 * pair + 1] = even * math.sin(angle) + odd * math.cos(angle)
    return out


def qk_case(rng, batch, tokens, d_model, num_heads, with_norm, rope_base, eps=1e-6):
    query = [[[dyadic(rng) for _ in range(d_model)] for _ in range(tokens)] for _ in range(batch)]
    key = [[[dyadic(rng) for _ in range(d_model)] for _ in range(tokens)] for _ in range(batch)]
    query_weight = [1.0 + dyadic(rng, 4, 8) for _ in range(d_model)] if with_norm else None
    key_weight = [1.0 + dyadic(rng, 4, 8) for _ in range(d_model)] if with_norm else None

    def transform(rows, weight):
        out = []
        for sample in rows:
            new_sample = []
            for position, row in enumerate(sample):
                values = rms_norm_row(row, weight, eps) if weight is not None else list(row)
                if rope_base is not None:
                    values = rotate_row(values, position, num_heads, rope_base)
                new_sample.append(values)
            out.append(new_sample)
        return out

    return {
        "num_heads": num_heads, "eps": eps, "rope_base": rope_base,
        "query": query, "key": key, "query_weight": query_weight, "key_weight": key_weight,
        "query_out": transform(query, query_weight), "key_out": transform(key, key_weight),
    }


def bag_case(rng, num_embeddings, emb_dim, bags, bag_size):
    weight = [[dyadic(rng) for _ in range(emb_dim)] for _ in range(num_embeddings)]
    values = [[rng.choice([0, 0] + list(range(1, num_embeddings))) for _ in range(bag_size)] for _ in range(bags)]
    values[0] = [0] * bag_size  # a bag of padding only
    values[1] = [values[1][0] or 1] * bag_size  # a bag that repeats one id
    out = []
    for bag in values:
        ids = [i for i in bag if i != 0]
        out.append([sum(weight[i][c] for i in ids) / max(1, len(ids)) for c in range(emb_dim)])
    return {"weight": weight, "values": values, "out": out}


def main() -> None:
    rng = random.Random(20260)
    payload = {
        "qk": [
            qk_case(rng, 2, 5, 16, 2, True, None),        # normalisation only
            qk_case(rng, 2, 5, 16, 2, True, 10000.0),     # normalisation + rotation, even head width
            qk_case(rng, 1, 7, 32, 4, False, 100.0),      # rotation only
            qk_case(rng, 2, 4, 40, 8, True, 10000.0),     # head width 5: the last feature of a head is not rotated
        ],
        "bags": [bag_case(rng, 9, 4, 6, 3), bag_case(rng, 17, 8, 5, 6)],
    }
    path = Path(__file__).resolve().parent / "qk_rope_embedding_small.json"
    path.write_text(json.dumps(payload) + "\n")
    print(f"wrote {path} ({path.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
