"""Writes tests/golden/fp8_transport_cases.json: the inputs of the reference's FP8 transport matrix and, for every
destination rank, what that rank must receive.

The reference builds these inputs from closed formulas and checks its dispatch against a gather written out in its own
test (tests/ascend/production/run_fp8_dispatch_combine.py:108-159 inputs, :228-305 expected rows, :373-396 the cached
representation changes, :398-425 the BF16 combine, :427-430 the 100 generations).  This script evaluates the same
formulas for world sizes 2 and 4 and records inputs and expected outputs as plain data, so that the tests need neither
the reference nor this script.  Run it from the repository root:  python tests/golden/make_fp8_transport_fixture.py

Layout of the file: worlds[W].cases[name] = {flags, sources[s] = inputs of source rank s, expected[d] = outputs of
destination rank d}.  A payload row is an index into row_table, whose entries are hex strings of the row's bytes (FP8: 1
byte a channel, BF16: 2, little endian; index 0 and 1 are the all-zero FP8 and BF16 rows); scale factors are the int32
bit patterns of each 4-byte pack, whatever their dtype.
"""
import json
import os

import torch

HIDDEN, NUM_TOPK, SF_PACKS, CAPACITY = 512, 2, 4, 4

ROW_TABLE = ["00" * HIDDEN, "00" * (2 * HIDDEN)]
ROW_INDEX = {row: i for i, row in enumerate(ROW_TABLE)}


def row_id(row_bytes):
    text = bytes(row_bytes).hex()
    if text not in ROW_INDEX:
        ROW_INDEX[text] = len(ROW_TABLE)
        ROW_TABLE.append(text)
    return ROW_INDEX[text]

#        name                  packed  col-major expanded zero-pad alignment weighted
FLAGS = {
    "normal-fp32":           (False, False, False, False, 1, False),
    "packed-int32":          (True,  True,  False, False, 1, False),
    "expanded":              (False, False, True,  False, 1, False),
    "zero-padded":           (False, True,  True,  True,  4, False),
    "weighted":              (False, False, False, False, 1, True),
    "empty-input":           (False, True,  False, False, 1, False),
    "asymmetric-routing":    (False, False, False, False, 1, False),
    "negative-one-route":    (False, False, False, False, 1, False),
}


def token_count(name, rank):
    if name == "empty-input":
        return 0
    if name == "asymmetric-routing":
        return 3 if rank == 0 else 1
    if name == "one-token":
        return 1
    return 2


def routes_of(name, rank, world, count):
    out = []
    for t in range(count):
        first = ((rank + t + 1) % world) * 2 + t % 2
        second = ((rank + t + 2) % world) * 2 + (t + 1) % 2
        if name == "negative-one-route":
            first, second = (-1 if t == 0 else first), -1
        out.append([first, second])
    return out


def source_inputs(name, rank, world, salt, fp8, packed, weighted):
    n = token_count(name, rank)
    values = torch.arange(n * HIDDEN, dtype=torch.float32).reshape(n, HIDDEN).remainder(31) - 15 + rank * 2 + salt
    x = values.to(torch.float8_e4m3fn if fp8 else torch.bfloat16).contiguous()
    src = {"x": [row_id(row.view(torch.uint8).tolist()) for row in x],
           "routes": routes_of(name, rank, world, n),
           "weights": None, "sf_bits": None}
    if weighted:
        w = (torch.arange(n * NUM_TOPK, dtype=torch.float32).reshape(n, NUM_TOPK) + 1 + rank) / 16
        src["weights"] = w.tolist()
    if fp8:
        if packed:
            # the pack of (token t, group g) counts up along tokens first: the reference hands it over transposed
            sf = (torch.arange(n * SF_PACKS, dtype=torch.int32).reshape(SF_PACKS, n) + 0x3F404142 + rank * 0x10101 + salt).T
        else:
            sf = ((torch.arange(n * SF_PACKS, dtype=torch.float32).reshape(n, SF_PACKS) + 1 + rank + salt) / 32).view(torch.int32)
        src["sf_bits"] = sf.tolist()
    return src


def align(v, a):
    return (v + a - 1) // a * a


def expected_for(dst, sources, fp8, expanded, alignment, weighted):
    """What destination rank dst holds after the dispatch: rows in (source rank, token) order; in expanded form one
    region per local expert, each starting at a multiple of the alignment, entries in (source, token, lane) order."""
    lo, hi = dst * 2, dst * 2 + 2
    incoming = [(s, t) for s, src in enumerate(sources) for t, route in enumerate(src["routes"])
                if any(lo <= e < hi for e in route)]
    out = {"rows": [list(r) for r in incoming]}
    if not expanded:
        out["payload"] = [sources[s]["x"][t] for s, t in incoming]
        out["sf_bits"] = [sources[s]["sf_bits"][t] for s, t in incoming] if fp8 else None
        out["topk"] = [[e - lo if lo <= e < hi else -1 for e in sources[s]["routes"][t]] for s, t in incoming]
        out["weights"] = [sources[s]["weights"][t] for s, t in incoming] if weighted else None
        return out
    counts = [0, 0]
    for s, t in incoming:
        for e in sources[s]["routes"][t]:
            if lo <= e < hi:
                counts[e - lo] += 1
    starts = [0, align(counts[0], alignment)]
    total = starts[1] + align(counts[1], alignment)
    payload = [0 if fp8 else 1] * total
    sf = [[0] * SF_PACKS for _ in range(total)] if fp8 else None
    weights = [0.0] * total if weighted else None
    valid = [False] * total
    seen = [0, 0]
    for s, t in incoming:
        for lane, e in enumerate(sources[s]["routes"][t]):
            if not lo <= e < hi:
                continue
            row = starts[e - lo] + seen[e - lo]
            seen[e - lo] += 1
            payload[row] = sources[s]["x"][t]
            valid[row] = True
            if fp8:
                sf[row] = sources[s]["sf_bits"][t]
            if weighted:
                weights[row] = sources[s]["weights"][t][lane]
    out.update(payload=payload, sf_bits=sf, topk=None, weights=weights, valid=valid,
               unaligned_counts=counts, aligned_counts=[starts[1], total - starts[1]])
    return out


def make_case(name, world, salt=0, fp8=True, flags=None, input_rule=None):
    packed, col_major, expanded, zero_pad, alignment, weighted = flags or FLAGS[name]
    rule = input_rule or name
    sources = [source_inputs(rule, r, world, salt, fp8, packed, weighted) for r in range(world)]
    return {"fp8": fp8, "packed_sf": packed, "column_major_output": col_major, "expanded": expanded,
            "zero_padding": zero_pad, "expert_alignment": alignment, "weighted": weighted, "salt": salt,
            "sources": sources,
            "expected": [expected_for(d, sources, fp8, expanded, alignment, weighted) for d in range(world)]}


def bf16_sum(values):
    """Contributions become BF16 first, are summed in FP32, and the sum becomes BF16 (:68-70)."""
    return float(torch.tensor(values, dtype=torch.bfloat16).to(torch.float32).sum().to(torch.bfloat16))


def make_combine(world):
    case = make_case("normal-fp32", world)
    fills = [[s * 100 + t * 10 + d + 1 for s, t in case["expected"][d]["rows"]] for d in range(world)]
    combined = []
    for s, src in enumerate(case["sources"]):
        per_token = []
        for t, route in enumerate(src["routes"]):
            dests = sorted({e // 2 for e in route if e >= 0})
            per_token.append(bf16_sum([s * 100 + t * 10 + d + 1 for d in dests]))
        combined.append(per_token)
    return {"dispatch": case, "fill_of_row": fills, "combined": combined}


def main():
    plain = (False, False, False, False, 1, False)
    packed = (True, False, False, False, 1, False)
    worlds = {}
    for world in (2, 4):
        cases = {name: make_case(name, world) for name in FLAGS}
        cached = [  # a handle made by one representation is reused by the other (:373-385)
            {"reuse_handle_of": None, **make_case("cached-bf16", world, salt=0, fp8=False, flags=plain)},
            {"reuse_handle_of": 0, **make_case("cached-fp8", world, salt=7, fp8=True, flags=packed)},
            {"reuse_handle_of": None, **make_case("cached-fp8", world, salt=11, fp8=True, flags=packed)},
            {"reuse_handle_of": 2, **make_case("cached-bf16", world, salt=13, fp8=False, flags=plain)},
        ]
        generations = [make_case("one-token", world, salt=s, flags=plain) for s in range(13)] if world == 2 else []
        worlds[str(world)] = {"num_experts": 2 * world, "cases": cases, "cached_sequence": cached,
                              "combine": make_combine(world), "generations_by_salt": generations}
    doc = {"_about": "Inputs and expected per-destination outputs of the reference's FP8 transport matrix "
                     "(tests/ascend/production/run_fp8_dispatch_combine.py) for world sizes 2 and 4. Data only; written by "
                     "tests/golden/make_fp8_transport_fixture.py.",
           "hidden": HIDDEN, "num_topk": NUM_TOPK, "sf_packs": SF_PACKS, "capacity": CAPACITY, "worlds": worlds,
           "row_table": ROW_TABLE}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fp8_transport_cases.json")
    with open(path, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
