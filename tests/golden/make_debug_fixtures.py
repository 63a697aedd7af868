"""Writes tests/golden/debug_graphs.json.

The reference ships no golden vectors; its two hand-written graphs ("debug" and
"debug_hetero", python/graphiler/utils/setup.py:41-42 and 73-81) are the closest
thing to fixtures.  This script evaluates every operator on them with plain
Python loops over exact rationals / Python floats (no numpy kernels, no oracle,
no reference import), so the vectors are independent of the code they check.
Inputs are small integers so every expected value is exactly representable.

Run:  python tests/golden/make_debug_fixtures.py
"""
import json
import math
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def group(n, key, other):
    pointer, nbr, eid = [0], [], []
    for v in range(n):
        for e, k in enumerate(key):
            if k == v:
                nbr.append(other[e])
                eid.append(e)
        pointer.append(len(nbr))
    return pointer, nbr, eid


def fixtures_for(name, n, src, dst, etype=None, n_etypes=0):
    e = len(src)
    in_ptr, in_nbr, in_eid = group(n, dst, src)
    out_ptr, out_nbr, out_eid = group(n, src, dst)
    F = 4
    x = [[(3 * v + 2 * f) % 7 - 3 for f in range(F)] for v in range(n)]      # node rows
    m = [[(5 * i + f) % 9 - 4 for f in range(F)] for i in range(e)]          # edge rows
    w = [(2 * i) % 5 - 2 for i in range(e)]                                  # edge scalars
    ul = [v - 1 for v in range(n)]
    vr = [2 * v + 1 for v in range(n)]
    fx = {"name": name, "num_nodes": n, "src": src, "dst": dst,
          "in_pointer": in_ptr, "in_node_indices": in_nbr, "in_edge_indices": in_eid,
          "out_pointer": out_ptr, "out_node_indices": out_nbr,
          "out_edge_indices": out_eid, "x": x, "m": m, "w": w, "ul": ul, "vr": vr}

    def rows(v):
        return range(in_ptr[v], in_ptr[v + 1])

    fx["copy_u_sum"] = [[sum(x[in_nbr[i]][f] for i in rows(v)) for f in range(F)]
                        for v in range(n)]
    fx["copy_e_sum"] = [[sum(m[in_eid[i]][f] for i in rows(v)) for f in range(F)]
                        for v in range(n)]
    fx["u_mul_e_sum"] = [[sum(x[in_nbr[i]][f] * w[in_eid[i]] for i in rows(v))
                          for f in range(F)] for v in range(n)]
    fx["dst_mul_e_sum"] = [[sum(x[out_nbr[i]][f] * w[out_eid[i]]
                                for i in range(out_ptr[v], out_ptr[v + 1]))
                            for f in range(F)] for v in range(n)]
    # max over in-edges; rows without in-edges hold -inf (written as null)
    fx["copy_u_max"] = [[max((x[in_nbr[i]][f] for i in rows(v)), default=None)
                         for f in range(F)] for v in range(n)]
    fx["u_add_v"] = [ul[src[i]] + vr[dst[i]] for i in range(e)]
    fx["u_dot_v"] = [sum(x[src[i]][f] * x[dst[i]][f] for f in range(F))
                     for i in range(e)]
    # edge softmax of the logits w over each destination's in-edges
    sm = [0.0] * e
    for v in range(n):
        ids = [in_eid[i] for i in rows(v)]
        if ids:
            mx = max(w[i] for i in ids)
            den = math.fsum(math.exp(w[i] - mx) for i in ids)
            for i in ids:
                sm[i] = math.exp(w[i] - mx) / den
    fx["edge_softmax_w"] = sm
    fx["gather_src"] = [x[s] for s in src]
    fx["gather_dst"] = [x[d] for d in dst]
    if etype is not None:
        K, M = F, 3
        W = [[[(t + 2 * k + 3 * j) % 5 - 2 for j in range(M)] for k in range(K)]
             for t in range(n_etypes)]
        fx["etype"] = etype
        fx["etype_pointer"] = [sum(1 for t in etype if t < r)
                               for r in range(n_etypes + 1)]
        fx["W"] = W
        fx["segment_mm_edge"] = [[sum(m[i][k] * W[etype[i]][k][j] for k in range(K))
                                  for j in range(M)] for i in range(e)]
    return fx


def main():
    out = [fixtures_for("debug", 3, [0, 0, 0, 1, 1, 2], [0, 1, 2, 1, 2, 2])]
    # debug_hetero flattened: users 0..2, movies 3..4, relations in listed order
    src = [0, 0, 1, 1, 2, 2, 0, 2, 3, 4]
    dst = [3, 4, 3, 4, 3, 4, 1, 1, 4, 3]
    et = [0, 0, 0, 1, 1, 1, 2, 3, 4, 5]
    out.append(fixtures_for("debug_hetero", 5, src, dst, et, 6))
    with open(os.path.join(HERE, "debug_graphs.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", len(out), "fixtures")


if __name__ == "__main__":
    main()
