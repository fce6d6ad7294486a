"""Writes tests/golden/fp8_gemm_golden.json: seeded inputs' checksums and sampled fp32 oracle outputs.

The reference holds no stored vectors for this path (its only test, tests/kernels/test_fp8_gemm.py, draws unseeded
random inputs on a GPU), so the fixture is produced by this repository's own CPU oracle; it pins the oracle and
the input generators against drift.  Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import torch  # noqa: E402

import helpers  # noqa: E402
from oracle import fp8_block_gemm as orc  # noqa: E402

CASES = [(64, 512, 1024, 20), (16, 2112, 1024, 21), (33, 200, 400, 22), (1, 130, 128, 23)]


def main():
    cases = []
    for M, N, K, seed in CASES:
        a_q, a_s, b_q, b_s = helpers.make_dense(M, N, K, seed=seed)
        ref = orc.dequant_ref(a_q, a_s, b_q, b_s)
        g = torch.Generator().manual_seed(seed)
        ms = torch.randint(0, M, (12, ), generator=g).tolist()
        ns = torch.randint(0, N, (12, ), generator=g).tolist()
        cases.append({
            'M': M, 'N': N, 'K': K, 'seed': seed,
            'a_q_bytesum': int(a_q.view(torch.uint8).long().sum()),
            'b_q_bytesum': int(b_q.view(torch.uint8).long().sum()),
            'sum': float(ref.double().sum()),
            'samples': [[m, n, float(ref[m, n])] for m, n in zip(ms, ns)],
        })
    with open(os.path.join(HERE, 'fp8_gemm_golden.json'), 'w') as fh:
        json.dump({'oracle': 'oracle/fp8_block_gemm.py:dequant_ref', 'cases': cases}, fh, indent=1)


if __name__ == '__main__':
    main()
