"""A whole logical world in one single-source call.

One dispatch call moves the tokens of ONE logical source rank.  To reproduce what every destination
rank of an R-rank run receives (the reference's own test setting) the tokens of source rank s are
placed at rows [s*M, s*M + n_s) of an R*M-row input whose other rows select nothing (-1).  Run as
source rank 0 with capacity R*M, the global source index rank*capacity + row equals s*M + t, the
index a real R-rank run reports, and destination bucket d lists its rows in (source rank, token)
order: exactly deep_ep/utils/refs.py:10-123.
"""
import json
import os

import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "two_rank_cases.json")


def load_golden():
    with open(GOLDEN) as f:
        return json.load(f)


def stack_world(payloads, routes, weights, M, hidden, num_topk):
    """Per-source lists -> (x[R*M, H] bf16, topk_idx[R*M, K] int64, topk_weights[R*M, K] fp32 or None)."""
    R = len(routes)
    x = torch.zeros((R * M, hidden), dtype=torch.bfloat16)
    idx = torch.full((R * M, num_topk), -1, dtype=torch.int64)
    w = torch.zeros((R * M, num_topk), dtype=torch.float32) if weights is not None else None
    for s in range(R):
        n = len(routes[s])
        if n == 0:
            continue
        idx[s * M:s * M + n] = torch.tensor(routes[s], dtype=torch.int64).view(n, num_topk)
        if payloads is not None:
            x[s * M:s * M + n] = torch.tensor(payloads[s], dtype=torch.float32).view(n, hidden).to(torch.bfloat16)
        if weights is not None:
            w[s * M:s * M + n] = torch.tensor(weights[s], dtype=torch.float32).view(n, num_topk)
    return x, idx, w


def per_source(x, idx, w, M, R, counts):
    """Inverse of stack_world: lists of per-source tensors."""
    xs = [x[s * M:s * M + counts[s]] for s in range(R)]
    idxs = [idx[s * M:s * M + counts[s]] for s in range(R)]
    ws = [None if w is None else w[s * M:s * M + counts[s]] for s in range(R)]
    return xs, idxs, ws


def bucket_bounds(psum_rank):
    ends = psum_rank.to(torch.int64).tolist()
    starts = [0] + ends[:-1]
    return list(zip(starts, ends))
