"""Writes the committed fixtures of tests/golden from the CPU oracle.

    python tests/golden/make_golden.py

fp8_tables.json : the 256-entry decode tables of fp_8bit<5,false> / <5,true> (fp32 and fp16 bit
                  patterns) and encode results for a spread of inputs.
toy_index.npz   : a 4-list, 64-row, dim-8 index (pq_dim 4, 8-bit) with queries and the oracle's
                  probes / neighbours / distances for the fp32 path; small enough to check by hand.
pack_cases.npz  : random codes and their interleaved list bytes for pq_bits 4..8.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle  # noqa: E402


def bits(f):
    return int(np.float32(f).view(np.uint32))


def main():
    L = oracle.lib()
    cases = []
    rng = np.random.default_rng(11)
    vals = np.concatenate([
        np.array([0.0, -1.0, 1.0, 1.2, -1.2, 2.0 ** -15, 2.0 ** -16, 122880.0, 1e9, 0.3, 77.7],
                 dtype=np.float32),
        np.exp(rng.uniform(np.log(1e-6), np.log(2e5), 200)).astype(np.float32),
        -np.exp(rng.uniform(np.log(1e-6), np.log(2e5), 50)).astype(np.float32)])
    for v in vals:
        cases.append([bits(v), int(L.orc_fp8_encode(float(v), 0)), int(L.orc_fp8_encode(float(v), 1))])
    gold = {
        "decode_unsigned_bits": [bits(L.orc_fp8_decode(u, 0)) for u in range(256)],
        "decode_signed_bits": [bits(L.orc_fp8_decode(u, 1)) for u in range(256)],
        "decode_half_unsigned_bits": [int(L.orc_fp8_decode_half(u, 0)) for u in range(256)],
        "encode_cases": cases,
    }
    with open(os.path.join(HERE, "fp8_tables.json"), "w") as f:
        json.dump(gold, f)

    # pack cases
    out = {}
    for pq_bits, pq_dim, n_rows in [(4, 8, 37), (5, 8, 70), (6, 12, 33), (7, 16, 5), (8, 20, 64)]:
        codes = rng.integers(0, 1 << pq_bits, (n_rows, pq_dim)).astype(np.uint8)
        out[f"codes_{pq_bits}"] = codes
        out[f"list_{pq_bits}"] = oracle.pack_list(codes, pq_bits)
    np.savez_compressed(os.path.join(HERE, "pack_cases.npz"), **out)

    # toy index
    dim, pq_dim, pq_bits, n_lists, n = 8, 4, 8, 4, 64
    data = rng.standard_normal((n, dim)).astype(np.float32)
    centers = data[rng.choice(n, n_lists, replace=False)].copy()
    padded = np.zeros((n_lists, oracle.dim_ext(dim)), dtype=np.float32)
    padded[:, :dim] = centers
    padded[:, dim] = (centers.astype(np.float32) ** 2).sum(1, dtype=np.float32)
    rot = np.eye(dim, dtype=np.float32)
    pq_centers = (rng.standard_normal((pq_dim, dim // pq_dim, 1 << pq_bits)) * 0.5).astype(np.float32)
    ix = oracle.Index(oracle.L2Expanded, oracle.PER_SUBSPACE, dim, pq_dim, pq_bits, padded,
                      centers.copy(), rot, pq_centers)
    labels, codes = oracle.encode(ix, data, n_threads=1)
    ix.fill(labels, codes)
    queries = rng.standard_normal((5, dim)).astype(np.float32)
    nb, dist, probes = oracle.search(ix, queries, 3, 2, n_threads=1, return_probes=True)
    np.savez_compressed(os.path.join(HERE, "toy_index.npz"), data=data, centers=padded,
                        pq_centers=pq_centers, labels=labels, codes=codes, queries=queries,
                        neighbors=nb, distances=dist, probes=probes)


if __name__ == "__main__":
    main()
