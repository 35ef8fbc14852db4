"""Extracts the worked vectors printed in the reference's python/ring_packing.ipynb into a JSON fixture.

The notebook is read as JSON text (its stored cell outputs); nothing of the reference is executed or imported.
Run in the build container only (the reference tree does not exist on the GPU box):
    python tests/golden/extract_notebook_vectors.py
Writes tests/golden/ring_packing_ipynb.json.
"""
import json
import os
import re

REF = "/root/reference/python/ring_packing.ipynb"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ring_packing_ipynb.json")


def parse_poly(s, n):
    """'3*xbar^2 + xbar + 7' -> coefficient list of length n."""
    co = [0] * n
    for term in s.strip().split(" + "):
        term = term.strip()
        if not term:
            continue
        m = re.fullmatch(r"(?:(\d+)\*)?xbar(?:\^(\d+))?", term)
        if m:
            c = int(m.group(1)) if m.group(1) else 1
            e = int(m.group(2)) if m.group(2) else 1
        else:
            c, e = int(term), 0
        co[e] = c
    return co


def main():
    nb = json.load(open(REF))
    out = lambda i: "".join(nb["cells"][i]["outputs"][0]["text"])
    fix = {"source": "python/ring_packing.ipynb stored outputs", "q": 65537}
    # cell 0: secret of the N=32 example
    fix["cell0_sx_big_ring"] = parse_poly(out(0).strip(), 32)
    lines = out(1).strip().split("\n")
    ax_down = lines[0][len("ax down ["):-1].split(", ")
    fix["cell1_ax_down"] = [parse_poly(p, 8) for p in ax_down]
    fix["cell1_ax_big_ring"] = parse_poly(lines[1][len("ax up "):], 32)
    fix["cell1_twist"] = parse_poly(lines[3][len("twist "):], 32)
    fix["cell1_twist_times_sx"] = parse_poly(lines[4], 32)
    fix["cell1_target"] = parse_poly(lines[5][len("target: "):], 8)
    fix["cell1_products"] = [parse_poly(lines[6 + i], 8) for i in range(4)]
    fix["cell1_inner_product"] = parse_poly(lines[10][len("inner product: "):], 8)
    # cell 6: (sum i x^i)^2 in Z_q[x]/(x^32+1) and its embedding in Z_q[x]/(x^256+1)
    l6 = out(6).strip().split("\n")
    fix["cell6_square_N256"] = parse_poly(l6[2], 256)
    fix["cell6_square_N32"] = parse_poly(l6[3], 32)
    json.dump(fix, open(OUT, "w"), indent=0)
    print("wrote", OUT)


if __name__ == "__main__":
    main()
