#!/usr/bin/env python3
"""Writes tests/golden/decode_graph_params.json: the argument list of the
reference's shipped decode graph
(/root/reference/examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:4) as
data -- index, shape and element type of every argument -- plus, for every
two-dimensional argument, how the graph's body uses it: as the weight of a plain
`linalg.matmul`, as the weight of a matmul whose result is added to a reshaped
one-dimensional argument (the decomposed AddMM: weight + bias), or not by a
matmul at all (the embedding table, read by a gather).

Reads the reference as text only; nothing of it is imported or run.

    python tests/golden/make_decode_graph_params.py
"""
import json
import re
import sys
from pathlib import Path

REF = Path("/root/reference/examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir")
OUT = Path(__file__).resolve().parent / "decode_graph_params.json"


def parse(text: str):
    lines = text.splitlines()
    head = next(l for l in lines if "func.func @subgraph0_decode(" in l)
    sig = head[head.index("("):head.index(") ->")]
    args = []
    for m in re.finditer(r"%arg(\d+): tensor<((?:\d+x)+)(f32|i64|i8)>", sig):
        args.append({"arg": int(m.group(1)),
                     "shape": [int(d) for d in m.group(2).rstrip("x").split("x")],
                     "dtype": m.group(3), "use": None, "bias": None})
    assert [a["arg"] for a in args] == list(range(len(args)))
    # %N = tosa.reshape %argK ...   (a parameter vector made a row)
    reshaped = {}
    for l in lines:
        m = re.match(r"\s*(%\w+) = tosa\.reshape %arg(\d+),", l)
        if m:
            reshaped[m.group(1)] = int(m.group(2))
    for i, l in enumerate(lines):
        m = re.match(r"\s*(%\w+) = linalg\.matmul .*ins\((%\w+), %arg(\d+) :", l)
        if not m:
            continue
        res, w = m.group(1), int(m.group(3))
        use, bias = "matmul", None
        for nxt in lines[i + 1:i + 4]:  # the bias add follows within three ops
            a = re.match(r"\s*%\w+ = tosa\.add (%\w+), (%\w+) :", nxt)
            if a and res in (a.group(1), a.group(2)):
                other = a.group(2) if a.group(1) == res else a.group(1)
                if other in reshaped:
                    use, bias = "addmm", reshaped[other]
        assert args[w]["use"] in (None, use)
        args[w]["use"], args[w]["bias"] = use, bias
    return args


def main():
    if not REF.exists():
        sys.exit(f"{REF} not found")
    args = parse(REF.read_text())
    OUT.write_text(json.dumps({"source": str(REF) + ":4", "args": args}, separators=(",", ":")))
    print(f"wrote {OUT}: {len(args)} arguments")


if __name__ == "__main__":
    main()
