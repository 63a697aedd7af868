#!/usr/bin/env python3
"""Per-operator timings at the other benchmark configurations (bench.py covers
configuration 2): one JSON line per operator with its algorithmic bytes, the
achieved algorithmic GB/s and, for the matrix products, TFLOP/s.

    python bench_kernels.py [c1] [c3] [c4] [c5]        # default: c1 c3 c4

  c1  GCN, 19,717 nodes / 108,368 edges: SpMM copy_u at F = 16 and 3
  c3  RGCN, 100 k nodes / 1 M edges / 60 relations: segment_mm 16->64 and 64->8
      (on per-edge rows and reading the source rows through the COO column),
      SpMM copy_e and e_mul_e, source gather, the whole layer (fp32 and bf16)
  c4  HGT, 100 k nodes / 2 M edges / 4 node types / 10 relations, 8 heads x 16:
      segment_mm on nodes and on edges (plain, gathered, with the dot-product
      epilogue), SDDMM u_dot_v, 8-head softmax, SpMM u_mul_e / e_mul_e, the layer
  c5  GAT, 2.45 M nodes / 64.3 M edges, 4 heads x 64 bf16: fused aggregation,
      SpMM u_mul_e, SDDMM u_add_v, 4-head softmax, the dense projection with its
      attention terms (100 -> 256 and 256 -> 256) beside the three ATen GEMMs it replaces

Inputs are resident on the device; each operator is timed with HIP events over
`--reps` calls after `--warmup` calls.  Byte counts credit one gathered row
per edge and no cache reuse, so a rate above the 8 TB/s memory peak means the
gathers were served from cache.
"""
import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("configs", nargs="*", default=["c1", "c3", "c4"])
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    args = ap.parse_args()

    import numpy as np
    import torch

    from graphiler_amd import datasets, layers, ops, prepare_graph

    if not torch.cuda.is_available():
        sys.exit("bench_kernels.py: no GPU visible")
    dev = "cuda:0"

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(args.reps):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / args.reps

    def report(config, name, fn, nbytes, flops=None):
        ms = timed(fn)
        line = {"config": config, "operator": name, "us": round(ms * 1e3, 1),
                "algorithmic_bytes": int(nbytes),
                "algorithmic_GBps": round(nbytes / ms / 1e6, 1)}
        if flops:
            line["TFLOPps"] = round(flops / ms / 1e9, 2)
        print(json.dumps(line), flush=True)

    def rnd(*shape, dtype=torch.float32):
        return torch.randn(*shape, device=dev).to(dtype)

    if "c1" in args.configs:
        wl = datasets.gcn_uniform()
        N, E = wl.num_nodes, wl.num_edges
        g = prepare_graph(wl.src, wl.dst, N, device=dev)
        g.in_row_of_slot
        for F in (16, 3):
            x = rnd(N, F)
            report("c1", f"spmm copy_u F={F} f32", lambda: ops.SpMMSrc(x, [1], False, None, g),
                   4 * (N + 1) + E * (4 + F * 4) + N * F * 4)

    if "c3" in args.configs:
        wl = datasets.rgcn_zipf()
        N, E, R = wl.num_nodes, wl.num_edges, wl.num_etypes
        g = prepare_graph(wl.src, wl.dst, N, device=dev, etype_of=wl.etype, num_etypes=R)
        g.in_row_of_slot
        for dt, b, tag in ((torch.float32, 4, "f32"), (torch.bfloat16, 2, "bf16")):
            for K, M in ((16, 64), (64, 8)):
                X, W = rnd(E, K, dtype=dt), rnd(R, K, M, dtype=dt)
                report("c3", f"segment_mm edge {K}->{M} {tag}", lambda: ops.SegmentMMEdge(X, W, g),
                       E * (K + M) * b + R * K * M * b, 2 * E * K * M)
                Xn = rnd(N, K, dtype=dt)
                report("c3", f"segment_mm gather src {K}->{M} {tag}",
                       lambda: ops.SegmentMMEdgeGather(Xn, W, 0, g),
                       E * (8 + (K + M) * b) + R * K * M * b, 2 * E * K * M)
            norm = torch.rand(E, 1, device=dev)
            for F in (64, 8):
                m = rnd(E, F, dtype=dt)
                report("c3", f"spmm copy_e F={F} {tag}", lambda: ops.SpMMEdge(m, [1], False, None, g),
                       4 * (N + 1) + E * (4 + 4 + F * b) + N * F * b)
                report("c3", f"spmm e_mul_e F={F} {tag}", lambda: ops.gspmm_e_mul_e_sum(m, norm, g),
                       4 * (N + 1) + E * (4 + 4 + 4 + F * b) + N * F * b)
            for K, M in ((16, 64), (64, 8)):
                Xn, W = rnd(N, K, dtype=dt), rnd(R, K, M, dtype=dt)
                for fused in (False, True):
                    report("c3", f"rgcn layer {K}->{M} {tag} {'fused' if fused else 'plan'}",
                           lambda: layers.rgcn_layer(g, Xn, W, norm, fused=fused),
                           4 * (N + 1) + E * (8 + 4 + 4 + K * b) + R * K * M * b + N * M * b,
                           2 * E * K * M)
        h = rnd(N, 16)
        report("c3", "gather src (N,16)->(E,16) f32", lambda: ops.BroadcastSrcNode(h, g),
               E * (8 + 64 + 64))

    if "c4" in args.configs:
        wl = datasets.hgt_hetero()
        N, E = wl.num_nodes, wl.num_edges
        g = prepare_graph(wl.src, wl.dst, N, device=dev, ntype_of=wl.ntype,
                          num_ntypes=wl.num_ntypes, etype_of=wl.etype, num_etypes=wl.num_etypes)
        g.in_row_of_slot
        dt, b, H, D = torch.bfloat16, 2, 8, 16
        X, W = rnd(N, 128, dtype=dt), rnd(wl.num_ntypes, 128, 128, dtype=dt)
        report("c4", "segment_mm node 128->128 bf16", lambda: ops.SegmentMMNode(X, W, g),
               N * 256 * b + wl.num_ntypes * 128 * 128 * b, 2 * N * 128 * 128)
        Xe, Wr = rnd(E, 128, dtype=dt), rnd(wl.num_etypes, H, D, D, dtype=dt)
        report("c4", "segment_mm edge 8 x (16->16) bf16", lambda: ops.SegmentMMEdge(Xe, Wr, g),
               E * 256 * b + wl.num_etypes * H * D * D * b, 2 * E * H * D * D)
        report("c4", "segment_mm gather src 8 x (16->16) bf16",
               lambda: ops.SegmentMMEdgeGather(X, Wr, 0, g),
               E * (8 + 512) + wl.num_etypes * H * D * D * b, 2 * E * H * D * D)
        report("c4", "segment_mm dot (src rows, dst rows) 8 x (16->16) bf16",
               lambda: ops.SegmentMMEdgeDot(X, Wr, 0, X, 1, g),
               E * (16 + 512 + 4 * H) + wl.num_etypes * H * D * D * b, 2 * E * H * D * D)
        q, k = rnd(N, H, D, dtype=dt), rnd(N, H, D, dtype=dt)
        report("c4", "sddmm u_dot_v 8x16 bf16", lambda: ops.gsddmm_u_dot_v(k, q, g),
               4 * (N + 1) + E * (4 + 2 * H * D * b + 4 * H))
        lg = rnd(E, H)
        report("c4", "segment_softmax H=8 f32", lambda: ops.SegmentSoftmax(lg, 1, None, g),
               4 * (N + 1) + 8 * E * H)
        a, v = torch.rand(E, H, device=dev), rnd(N, H * D, dtype=dt)
        report("c4", "spmm u_mul_e H=8 F=128 bf16",
               lambda: ops.gspmm_src_mul_e_sum(v, a, [1], False, None, g),
               4 * (N + 1) + E * (4 + 4 * H + H * D * b) + N * H * D * b)
        report("c4", "spmm e_mul_e H=8 F=128 bf16", lambda: ops.spmm(g, "e_mul_e", "sum", Xe, a),
               4 * (N + 1) + E * (4 + 4 + 4 * H + H * D * b) + N * H * D * b)
        report("c4", "gather src (N,128)->(E,128) bf16", lambda: ops.BroadcastSrcNode(X, g),
               E * (8 + 256 + 256))
        wk, wq, wv, wa = (rnd(wl.num_ntypes, 128, 128, dtype=dt) / 11 for _ in range(4))
        ra, rm = (rnd(wl.num_etypes, H, D, D, dtype=dt) / 4 for _ in range(2))
        rp = torch.rand(wl.num_etypes, H, device=dev).to(dt)
        skip = torch.ones(wl.num_ntypes, device=dev)
        # bytes of the fused layer: h in, K/V/Q/t/out node rows, three gathered
        # rows per edge, the transformed values written and read once, scores
        layer_bytes = N * 128 * b * 9 + E * (3 * 128 * b + 2 * 128 * b + 24 + 6 * 4 * H)
        for fused in (False, True):
            report("c4", f"hgt layer bf16 {'fused' if fused else 'plan'}",
                   lambda: layers.hgt_layer(g, X, wk, wq, wv, wa, ra, rm, rp, skip, H, fused=fused),
                   layer_bytes, 2 * N * 128 * 128 * 4 + 4 * E * H * D * D)

    if "c5" in args.configs:
        wl = datasets.gat_rmat_large()
        N, E = wl.num_nodes, wl.num_edges
        g = prepare_graph(wl.src, wl.dst, N, device=dev)
        g.in_row_of_slot
        dt, b, H, F = torch.bfloat16, 2, 4, 256
        z, el, er = rnd(N, F, dtype=dt), rnd(N, H), rnd(N, H)
        report("c5", "gat_aggregate H=4 F=256 bf16", lambda: ops.gat_aggregate(el, er, z, g, 0.2),
               4 * (N + 1) + E * (4 + H * 4 + F * b) + N * (H * 4 + F * b))
        a_l = rnd(H, F // H) / 8
        report("c5", "gat_aggregate, source term from z, H=4 F=256 bf16",
               lambda: ops.gat_aggregate_from_z(a_l, er, z, g, 0.2),
               4 * (N + 1) + E * (4 + F * b) + N * (H * 4 + F * b))
        a = torch.rand(E, H, device=dev)
        report("c5", "spmm u_mul_e H=4 F=256 bf16",
               lambda: ops.gspmm_src_mul_e_sum(z, a, [1], False, None, g),
               4 * (N + 1) + E * (4 + 4 * H + F * b) + N * F * b)
        report("c5", "sddmm u_add_v H=4 f32", lambda: ops.gsddmm_u_add_v_mul_alpha(el, er, 1, g),
               4 * (N + 1) + E * (4 + H * 4 + 4 * H) + N * H * 4)
        lg = rnd(E, H)
        report("c5", "segment_softmax H=4 f32", lambda: ops.SegmentSoftmax(lg, 1, None, g),
               4 * (N + 1) + 8 * E * H)
        # the whole three-layer network (100 -> 256 -> 256 -> 256, 4 heads x 64, elu
        # between layers) compiled from its user-defined functions
        from graphiler_amd.examples import udf
        from graphiler_amd.mpdfg import GraphData, mpdfg_builder, update_all
        plan = mpdfg_builder(udf.gat4x64_message, udf.gat4_reduce, opt_level=2)
        gd = GraphData(g)
        x0 = rnd(N, 100, dtype=dt)
        params = [(rnd(k, F, dtype=dt) / 16, rnd(1, H, F // H) / 8, rnd(1, H, F // H) / 8)
                  for k in (100, F, F)]

        def network():
            x = x0
            for fc, a_l, a_r in params:
                gd.ndata["h"] = x
                out = update_all(gd, plan, msg_params=(fc, a_l, a_r))["h"]
                x = torch.nn.functional.elu(out).view(N, F)
            return x

        layer_bytes = lambda k: (N * (k + F) * b + k * F * b +
                                 4 * (N + 1) + E * (4 + F * b) + N * (H * 4 + F * b))
        report("c5", "3-layer GAT compiled from UDFs (gat_project_heads + gat_aggregate_al per layer)",
               network, sum(layer_bytes(k) for k in (100, F, F)),
               sum(2 * N * k * F for k in (100, F, F)))
        al, ar = rnd(H, F // H), rnd(H, F // H)
        bl, br = rnd(F, H, dtype=dt), rnd(F, H, dtype=dt)     # block-diagonal (F, H) forms
        for K in (100, 256):          # first and hidden layers
            x, w = rnd(N, K, dtype=dt), rnd(K, F, dtype=dt) / 16
            report("c5", f"projection + attention terms {K}->256 bf16",
                   lambda: ops.linear_attn(x, w, al, ar),
                   N * (K + F) * b + K * F * b + 2 * N * H * 4, 2 * N * K * F + 4 * N * F)
            report("c5", f"three ATen GEMMs {K}->256 bf16 (z, el, er)",
                   lambda: (lambda z: (z, z @ bl, z @ br))(x @ w),
                   N * (K + F) * b + K * F * b + 2 * N * H * 4, 2 * N * K * F + 4 * N * F)


if __name__ == "__main__":
    main()
