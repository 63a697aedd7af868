#!/usr/bin/env python3
"""Benchmark of the graph-primitive layer on one MI355X: GAT / RGCN / HGT layer
forwards at the benchmark configurations, with per-kernel roofline figures.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs c5,c2,c3,c4,c1]
                    [--only KEY[,KEY]] [--no-cpu-baseline] [--markers]

Headline (the JSON line's metric / value / roofline / cpu_baseline): the first
configuration named in --configs, by default c5 = configs[4], the largest one
that fits one GPU: 3-layer GAT, 4 heads x 64, bf16 features with fp32 softmax and
accumulation, R-MAT graph with 2,449,029 nodes and 64,308,169 edges.  A step is one
forward pass of the whole network (100 -> 256 -> 256 -> 256: per layer the dense
projection with its attention terms, then the fused chain u_add_v -> leaky_relu ->
edge softmax -> u_mul_e sum, elu between layers); `value` counts the edges the three
layers traverse per second.  All inputs are resident in HBM before the timed region.

The other configurations (c2 = configs[1] 1-head fp32 GAT, c3 = configs[2] RGCN
fp32 and bf16, c4 = configs[3] HGT bf16, c1 = configs[0] the 2-layer GCN that the
configuration list assigns to the host cores, timed there and on the GPU) are measured
in the same run and reported as objects under "configs" of the same line: layer time, edges/s and, per operator,
launch time (HIP events on the launch stream), algorithmic bytes, effective GB/s,
fraction of the 8 TB/s HBM peak and, for the matrix kernels, TFLOP/s against the
MFMA peak and against min(MFMA peak, intensity x HBM peak).

Algorithmic bytes credit one gathered row per edge and no cache reuse.  An operator
whose gathered table fits the 256 MB Infinity Cache, or whose algorithmic bytes flow
faster than the HBM peak, is marked "cache_served": its fraction is then taken from the
L2 <-> fabric traffic that rocprofv3 counted for the operator's own dispatches (read
from profiles/hbm_traffic.md, separate counter runs of this script with --markers: not
measured here), and is null when no such count exists.  A count below the bytes the
operator writes cannot be that operator's and is refused.

--markers brackets every timed operator with an elementwise pass over 1 GiB
(`x.add(0)`: reads 1 GiB, writes 1 GiB).  In a rocprofv3 trace or counter file the
dispatches between two such passes are exactly one operator's calls (the line's
"profile_segments" lists key and number of calls in order), and the passes themselves
calibrate the counters.
Prints ONE JSON line.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                                   # MI355X published HBM3E bandwidth
INFINITY_CACHE_BYTES = 256 << 20                        # memory-side cache in front of the HBM
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}       # published dense matrix peaks
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.md")


def load_traffic():
    """{key: bytes per call} from the table rows `| key | fetch KiB | write KiB | bytes |`
    of profiles/hbm_traffic.md; empty when the file is absent."""
    table = {}
    if os.path.exists(TRAFFIC_FILE):
        for line in open(TRAFFIC_FILE):
            m = re.match(r"\|\s*`?([a-z0-9_.]+)`?\s*\|[^|]*\|[^|]*\|\s*([0-9,]+)\s*\|", line)
            if m:
                table[m.group(1)] = int(m.group(2).replace(",", ""))
    return table


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--configs", default="c5,c2,c3,c4,c1",
                    help="comma-separated subset of c1,c2,c3,c4,c5; the first one is the headline")
    ap.add_argument("--only", default="",
                    help="comma-separated operator keys (c4.hgt_layer, c2.segment_softmax, ...): time "
                         "only these, skip the network steps and the CPU legs (short profiler runs)")
    ap.add_argument("--reps", type=int, default=30, help="timed calls per operator")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--gather-ceiling", "--reference-points", dest="gather_ceiling", action="store_true",
                    help="configs[4]: also run its aggregation kernels on graphs with the same "
                         "destinations and uniformly random sources over tables of several sizes (HBM, "
                         "Infinity Cache, L2): what the memory system gives a gather of 512-byte rows; "
                         "configs[1] and [4]: u_add_v next to plain gathers of the same rows (torch's "
                         "index_select, the library's BroadcastSrcNode) and the write of its result alone, "
                         "and the segment softmax on regular segments of 64 next to torch.softmax over the "
                         "same view and a copy of the tensor")
    ap.add_argument("--no-ops", action="store_true",
                    help="time the layers only (shorter kernel traces for profiling)")
    ap.add_argument("--markers", "--calibrate-copy", dest="markers", action="store_true",
                    help="bracket every timed operator with an elementwise pass over 1 GiB (x.add(0)): "
                         "segment boundaries and counter calibration for rocprofv3 runs")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus must be 1 "
                 "(the path is not sharded across devices)")
    wanted = [c for c in args.configs.split(",") if c]
    for c in wanted:
        if c not in ("c1", "c2", "c3", "c4", "c5"):
            sys.exit(f"bench.py: unknown configuration {c!r}")

    import numpy as np
    import torch
    import torch.nn.functional as F

    from graphiler_amd import datasets, layers, ops, prepare_graph

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    traffic = load_traffic()
    only = {k for k in args.only.split(",") if k}
    if only:
        args.no_cpu_baseline = True
    segments = []                      # (key, calls) of every bracketed operator, in order
    marker_buf = torch.zeros(1 << 28, dtype=torch.float32, device=dev) if args.markers else None

    def marker():
        if marker_buf is not None:
            marker_buf.add(0.0)        # reads 1 GiB, writes 1 GiB (the result is dropped)

    def u_add_v_reference(g_, el_, er_, src_host):
        """--gather-ceiling: u_add_v next to gathers of the same (N, H) rows by the same source ids
        alone -- torch's index_select (the vendor's kernel) and the library's BroadcastSrcNode --
        and next to the write of the (E, H) result alone."""
        e_, h_ = g_.num_edges, int(el_.shape[1])
        src_ = torch.from_numpy(src_host).to(dev)
        out_ = torch.empty(e_, h_, device=dev)
        return {"rows": e_, "row_bytes": h_ * 4, "table_MB": round(el_.numel() * 4 / 1e6, 2),
                "u_add_v_ms": round(ev_time(lambda: ops.gsddmm_u_add_v_mul_alpha(el_, er_, 1, g_), 10), 4),
                "gather_alone_ms": round(ev_time(lambda: ops.BroadcastSrcNode(el_, g_), 10), 4),
                "torch_index_select_ms": round(ev_time(lambda: torch.index_select(el_, 0, src_, out=out_), 5), 4),
                "write_alone_ms": round(ev_time(lambda: out_.copy_(el_[:1].expand(e_, h_)), 10), 4)}

    def softmax_reference(g_, heads_):
        """--reference-points: the segment softmax of the graph's (E, H) logits next to the same
        number of logits in regular segments of 64 -- through the library and through torch.softmax
        over the (E / 64, 64, H) view, which knows the segments from the shape -- and next to a
        copy of the tensor (what reading and writing it once costs)."""
        e_ = g_.num_edges
        x_ = torch.randn(e_, heads_, device=dev)
        e64 = e_ - e_ % 64
        reg = prepare_graph(np.zeros(e64, np.int64), np.repeat(np.arange(e64 // 64), 64), e64 // 64,
                            device=dev)
        reg.in_row_of_slot
        xr, y_ = x_[:e64].contiguous(), torch.empty_like(x_)
        out = {"logits": e_ * heads_,
               "graph_ms": round(ev_time(lambda: ops.SegmentSoftmax(x_, 1, None, g_), 10), 4),
               "regular_segments_of_64_ms": round(ev_time(lambda: ops.SegmentSoftmax(xr, 1, None, reg), 10), 4),
               "torch_softmax_regular_segments_of_64_ms":
                   round(ev_time(lambda: torch.softmax(xr.view(-1, 64, heads_), dim=1), 5), 4),
               "copy_ms": round(ev_time(lambda: y_.copy_(x_), 10), 4)}
        out["regular_frac_of_8TBps"] = round(8.0 * e64 * heads_ / out["regular_segments_of_64_ms"] / 1e6 / HBM_PEAK_GBS, 4)
        return out

    def ev_time(fn, reps=None, warmup=3, key=None):
        reps = reps or args.reps
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        if key is not None:
            marker()
        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            fn()
        e.record()
        if key is not None:
            marker()
            segments.append([key, reps])
        torch.cuda.synchronize()
        return s.elapsed_time(e) / reps

    def wall_time(fn, steps, warmup, key=None):
        """Wall-clock time per call of a network step (None with --only: steps are
        not operators of their own)."""
        if only:
            return None, fn()
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        marker()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = fn()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        marker()
        if key is not None:
            segments.append([key, steps])
        return dt * 1e3 / steps, out

    def tensor_bytes(out):
        if isinstance(out, torch.Tensor):
            return out.numel() * out.element_size()
        return sum(tensor_bytes(o) for o in out) if isinstance(out, (tuple, list)) else 0

    def op_record(key, fn, nbytes, flops=None, mfma=None, reps=None, gather=None):
        """Launch time and roofline position of one operator call.  ``gather`` = (bytes of
        the table the operator gathers rows from, bytes of gathered rows among ``nbytes``);
        None for an operator that streams."""
        if only and key not in only:
            return None
        written = tensor_bytes(fn())
        ms = ev_time(fn, reps, key=key)
        gbps = nbytes / ms / 1e6
        rec = {"ms": round(ms, 4), "algorithmic_bytes": int(nbytes), "written_bytes": int(written),
               "effective_GBps": round(gbps, 1), "frac_algorithmic": round(gbps / HBM_PEAK_GBS, 4),
               "bound": "hbm"}
        moved = traffic.get(key)
        if moved is not None and moved < 0.98 * written:
            rec["traffic_refused"] = ("the recorded count (%d B) is below the %d B this operator "
                                      "writes: not this operator's dispatches" % (moved, written))
            moved = None
        if moved is not None:
            rec["traffic"] = moved
            rec["traffic_GBps"] = round(moved / ms / 1e6, 1)
        cached_table = gather is not None and gather[0] <= INFINITY_CACHE_BYTES \
            and 2 * gather[1] >= nbytes
        if gbps > HBM_PEAK_GBS or cached_table:
            # most of the algorithmic bytes are rows gathered from a table that the L2s and
            # the Infinity Cache hold: bytes over time is not memory bandwidth.  The fraction
            # is the counted L2 <-> fabric traffic (itself an upper bound of the HBM traffic:
            # Infinity Cache hits are counted), and never more than the algorithmic figure
            rec["cache_served"] = True
            rec["frac"] = round(min(moved, nbytes) / ms / 1e6 / HBM_PEAK_GBS, 4) if moved else None
            rec["frac_basis"] = "min(counted traffic, algorithmic bytes)" if moved else None
        else:
            rec["frac"] = rec["frac_algorithmic"]
            rec["frac_basis"] = "algorithmic bytes"
        if flops:
            peak = MFMA_PEAK_TFLOPS[mfma]
            tf = flops / ms / 1e9
            ceiling = min(peak, flops / nbytes * HBM_PEAK_GBS / 1e3)
            rec.update({"mfma_tflops": round(tf, 2), "mfma_peak_tflops": peak,
                        "mfma_util": round(tf / peak, 4),
                        "ceiling_tflops": round(ceiling, 1),
                        "frac_of_ceiling": round(tf / ceiling, 4)})
        return rec

    def kept(table):
        return {k: v for k, v in table.items() if v is not None}

    def per_s(count, ms):
        return None if ms is None else round(count / (ms * 1e-3), 1)

    def r4(ms, div=1):
        return None if ms is None else round(ms / div, 4)

    def cpu_time(fn, budget_s=10.0, min_reps=3, max_reps=50):
        """One warm-up pass, then at least ``min_reps`` timed passes (more while they fit
        ``budget_s``); returns (ms per pass, passes, last result)."""
        fn()
        reps, t0 = 0, time.perf_counter()
        while reps < min_reps or (time.perf_counter() - t0 < budget_s and reps < max_reps):
            out = fn()
            reps += 1
        return (time.perf_counter() - t0) * 1e3 / reps, reps, out

    def rnd(*shape, dtype=torch.float32, scale=1.0):
        return (torch.randn(*shape, device=dev) * scale).to(dtype)

    def copy_rate():
        """Device-to-device copy of 1 GiB: the practical ceiling of a streaming kernel."""
        a = torch.empty(1 << 28, dtype=torch.float32, device=dev)
        b = torch.empty_like(a)
        ms = ev_time(lambda: b.copy_(a), reps=20)
        del a, b
        return round(2 * (1 << 30) / ms / 1e6, 1)

    results = {}
    cpu = None
    headline = wanted[0]

    # ------------------------------------------------------------------ c5 ----
    def run_c5():
        nonlocal cpu
        wl = datasets.gat_rmat_large()                      # configs[4], seed 4
        N, E = wl.num_nodes, wl.num_edges
        g = prepare_graph(wl.src, wl.dst, N, device=dev)
        g.in_row_of_slot                                    # per-graph schedule, built once
        assert g.in_eid_is_identity
        max_deg = int(torch.diff(g.in_pointer).max().item())
        H, D, slope = 4, 64, 0.2
        Fw = H * D
        dt, b = torch.bfloat16, 2
        rng = np.random.default_rng(4)
        x0_h = rng.standard_normal((N, 100), dtype=np.float32)
        params_h = [(datasets.glorot(rng, (k, Fw)),
                     datasets.glorot(rng, (2, H, D), fan_in=2 * D, fan_out=1)) for k in (100, Fw, Fw)]
        x0 = torch.from_numpy(x0_h).to(dev).to(dt)
        params = [(torch.from_numpy(w).to(dev).to(dt), torch.from_numpy(a).to(dev))
                  for w, a in params_h]

        def network():
            x = x0
            for w, a in params:
                # F.elu between the layers, none after the last (examples/GAT/GAT.py:80-84)
                x = layers.gat_layer(g, x, w, a, H, slope, fused=True,
                                     activation=None if w is params[-1][0] else "elu")
            return x

        ms_step, out = wall_time(network, args.steps, args.warmup, key="c5.step")
        # the same steps once more with HIP events around every launch of the dominant
        # operator (on the stream it is launched on): its duration inside the network.  A
        # pass of its own because the event records cost 0.2 ms per step, which the timed
        # steps above should not pay
        inside = []
        plain_from_z = ops.gat_aggregate_from_z

        def timed_from_z(*a, **kw):
            s_ev = torch.cuda.Event(enable_timing=True)
            e_ev = torch.cuda.Event(enable_timing=True)
            s_ev.record()
            r = plain_from_z(*a, **kw)
            e_ev.record()
            inside.append((s_ev, e_ev))
            return r

        if not only:
            ops.gat_aggregate_from_z = timed_from_z
            try:
                for _ in range(args.steps):
                    network()
                torch.cuda.synchronize()
            finally:
                ops.gat_aggregate_from_z = plain_from_z
        inside = [s_ev.elapsed_time(e_ev) for s_ev, e_ev in inside]
        rec = {"workload": "configs[4]: 3-layer GAT 100->256->256->256, 4 heads x 64, bf16 features, "
                           "fp32 softmax and accumulation; R-MAT(a=.57,b=.19,c=.19, seed 4) + self loops",
               "num_nodes": N, "num_edges": E, "max_in_degree": max_deg, "dtype": "bf16",
               "ms_per_step": r4(ms_step), "ms_per_layer": r4(ms_step, 3),
               "edges_per_s": per_s(3 * E, ms_step)}
        z, el, er = layers.gat_project(x0, *params[0], H)
        z1, el1, er1 = layers.gat_project(z, *params[1], H)
        a_l = params[1][1][0].contiguous()
        fused_bytes = 4 * (N + 1) + E * (4 + Fw * b) + N * (H * 4 + Fw * b)
        opsr = {}
        opsr["gat_aggregate_from_z"] = op_record(
            "c5.gat_aggregate_from_z", lambda: ops.gat_aggregate_from_z(a_l, er1, z1, g, slope),
            fused_bytes, gather=(N * Fw * b, E * Fw * b))
        if not args.no_ops:
            opsr["gat_aggregate"] = op_record(
                "c5.gat_aggregate", lambda: ops.gat_aggregate(el1, er1, z1, g, slope),
                4 * (N + 1) + E * (4 + H * 4 + Fw * b) + N * (H * 4 + Fw * b),
                gather=(N * Fw * b, E * Fw * b))
            att = torch.rand(E, H, device=dev)
            opsr["spmm_u_mul_e"] = op_record(
                "c5.spmm_u_mul_e", lambda: ops.gspmm_src_mul_e_sum(z1, att, [1], False, None, g),
                4 * (N + 1) + E * (4 + 4 * H + Fw * b) + N * Fw * b, gather=(N * Fw * b, E * Fw * b))
            opsr["sddmm_u_add_v"] = op_record(
                "c5.sddmm_u_add_v", lambda: ops.gsddmm_u_add_v_mul_alpha(el1, er1, 1, g),
                4 * (N + 1) + E * (4 + H * 4 + 4 * H) + N * H * 4, gather=(N * H * 4, E * H * 4))
            lg = rnd(E, H)
            opsr["segment_softmax"] = op_record(
                "c5.segment_softmax", lambda: ops.SegmentSoftmax(lg, 1, None, g),
                4 * (N + 1) + 8 * E * H)
            del att, lg
            for k, (w, a) in ((100, params[0]), (256, params[1])):
                xin = x0 if k == 100 else z
                opsr[f"project_attn_{k}_256"] = op_record(
                    f"c5.project_attn_{k}_256", lambda: layers.gat_project(xin, w, a, H),
                    N * (k + Fw) * b + k * Fw * b + 2 * N * H * 4,
                    2.0 * N * k * Fw + 4.0 * N * Fw, "bf16")
        rec["ops"] = opsr = kept(opsr)
        if "gat_aggregate_from_z" in opsr:
            roof = dict(opsr["gat_aggregate_from_z"], kernel="gat_aggregate_from_z "
                        "(runs_kernel<GatPolicy<bf16, 8, from z>> + fix-up)")
            if inside:
                # the headline figure is the operator's duration inside the network steps;
                # "ms_back_to_back" keeps the repetitions of the operator on its own (its hot
                # rows still in the Infinity Cache from the call before)
                ms_in = sum(inside) / len(inside)
                roof.update({"ms_back_to_back": roof["ms"], "ms": round(ms_in, 4),
                             "launches_timed": len(inside),
                             "effective_GBps": round(fused_bytes / ms_in / 1e6, 1),
                             "frac": round(fused_bytes / ms_in / 1e6 / HBM_PEAK_GBS, 4),
                             "frac_algorithmic": round(fused_bytes / ms_in / 1e6 / HBM_PEAK_GBS, 4)})
                if "traffic" in roof:
                    roof["traffic_GBps"] = round(roof["traffic"] / ms_in / 1e6, 1)
            rec["roofline"] = roof
        if "project_attn_256_256" in opsr:
            rec["mfma"] = dict(opsr["project_attn_256_256"], kernel="project_attn 256 -> 256 bf16 "
                               "(wide_mm_kernel, v_mfma_f32_16x16x32_bf16)")

        if args.gather_ceiling and not only:
            # the same destinations, sources drawn uniformly from the first K rows of z: K = N
            # misses every cache (the random-row rate of the HBM), 2^17 rows = 67 MB stay in the
            # Infinity Cache, 2^13 rows = 4 MB in an L2 (what the kernel's own instructions allow)
            ceil = {}
            crng = np.random.default_rng(44)
            for K in (N, 1 << 17, 1 << 13):
                gk = prepare_graph(crng.integers(0, K, E), wl.dst, N, device=dev)
                gk.in_row_of_slot
                t_z = ev_time(lambda: ops.gat_aggregate_from_z(a_l, er1, z1, gk, slope), 10)
                t_c = ev_time(lambda: ops.SpMMSrc(z1, [1], False, None, gk), 10)
                ceil[f"uniform_sources_over_{K}_rows"] = {
                    "table_MB": round(K * Fw * b / 1e6, 1),
                    "gat_aggregate_from_z_ms": round(t_z, 4),
                    "gat_aggregate_from_z_row_GBps": round(E * Fw * b / t_z / 1e6, 1),
                    "spmm_copy_u_ms": round(t_c, 4),
                    "spmm_copy_u_row_GBps": round(E * Fw * b / t_c / 1e6, 1)}
                del gk
                torch.cuda.empty_cache()
            rec["gather_ceiling"] = ceil
            rec["u_add_v_reference"] = u_add_v_reference(g, el1.float().contiguous(), er1.float().contiguous(), wl.src)
            rec["softmax_reference"] = softmax_reference(g, H)

        if headline == "c5" and not args.no_cpu_baseline:
            # one hidden layer (256 -> 256) of the same network on the host cores: the fp32
            # C port of the reference's operators + torch-CPU projection
            import oracle
            ptr = g.in_pointer.cpu().numpy()
            nbr = g.in_node_indices.cpu().numpy()
            xin = z.float().cpu()
            w_f = params[1][0].float().cpu()
            a_f = params[1][1].cpu().numpy()

            def cpu_layer():
                zc = torch.mm(xin, w_f).numpy()
                zh = zc.reshape(N, H, D)
                elc = (zh * a_f[0]).sum(-1).astype(np.float32)
                erc = (zh * a_f[1]).sum(-1).astype(np.float32)
                lg_ = oracle.sddmm_u_add_v(wl.src, wl.dst, elc, erc)
                lg_ = np.where(lg_ >= 0, lg_, np.float32(slope) * lg_).astype(np.float32)
                at = oracle.segment_softmax(ptr, None, lg_, zero_floor=True)
                return oracle.spmm_sum_f32(ptr, nbr, None, zc, at, op="u_mul_e", heads=H)

            cpu_ms, cpu_reps, ref = cpu_time(cpu_layer)
            got = layers.gat_layer(g, z, params[1][0], params[1][1], H, slope).float().cpu().numpy()
            err = float(np.abs(got - ref).max() / np.abs(ref).max())
            cpu = {"value": round(E / (cpu_ms * 1e-3), 1), "unit": "edges/s",
                   "cores": oracle.num_threads(), "kind": "port",
                   "ms_per_layer": round(cpu_ms, 1),
                   "passes": cpu_reps,
                   "sample": f"one hidden layer (256 -> 256, all {E} edges, 4 heads) of the "
                             f"3-layer network: one warm-up pass, then the mean of {cpu_reps} passes of "
                             "the fp32 C port (OpenMP) of the four graph operators + torch-CPU projection",
                   "max_rel_diff_vs_gpu_bf16": err}
        return rec

    # ------------------------------------------------------------------ c2 ----
    def run_c2():
        nonlocal cpu
        wl = datasets.gat_rmat()                            # configs[1], seed 1
        N, E = wl.num_nodes, wl.num_edges
        g = prepare_graph(wl.src, wl.dst, N, device=dev)
        g.in_row_of_slot
        in_dim, Fw, H, slope, b = 602, 64, 1, 0.2, 4
        rng = np.random.default_rng(1)
        x_h = rng.standard_normal((N, in_dim), dtype=np.float32)
        w_h = datasets.glorot(rng, (in_dim, Fw))
        a_h = datasets.glorot(rng, (2, H, Fw // H), fan_in=2 * Fw, fan_out=1)
        x, w, a = (torch.from_numpy(t).to(dev) for t in (x_h, w_h, a_h))
        ms_step, out = wall_time(lambda: layers.gat_layer(g, x, w, a, H, slope, fused=True),
                                 max(args.steps, 100), max(args.warmup, 10), key="c2.step")
        rec = {"workload": "configs[1]: 1-head GAT layer 602->64 fp32 (dense projection + fused "
                           "chain); R-MAT(a=.57,b=.19,c=.19, seed 1)",
               "num_nodes": N, "num_edges": E, "dtype": "f32",
               "ms_per_step": r4(ms_step), "edges_per_s": per_s(E, ms_step)}
        z, el, er = layers.gat_project(x, w, a, H)
        rows = (N * Fw * b, E * Fw * b)
        opsr = {}
        opsr["gat_aggregate"] = op_record(
            "c2.gat_aggregate", lambda: ops.gat_aggregate(el, er, z, g, slope),
            4 * (N + 1) + E * (4 + H * b + Fw * b) + N * (H * b + Fw * b), reps=50, gather=rows)
        dense_bytes = 4 * (N * in_dim + in_dim * Fw + N * Fw + 2 * N * H)
        opsr["linear_attn_602_64"] = op_record(
            "c2.linear_attn", lambda: layers.gat_project(x, w, a, H), dense_bytes, reps=50)
        if opsr["linear_attn_602_64"] is not None:
            dms = opsr["linear_attn_602_64"]["ms"]
            opsr["linear_attn_602_64"]["fp32_equivalent_tflops"] = round(2.0 * N * in_dim * Fw / dms / 1e9, 2)
            opsr["linear_attn_602_64"]["bf16_piece_mfma_tflops"] = round(12.0 * N * in_dim * Fw / dms / 1e9, 1)
        if not args.no_ops:
            logits = F.leaky_relu_(ops.gsddmm_u_add_v_mul_alpha(el, er, 1, g), slope)
            att = ops.SegmentSoftmax(logits, 1, None, g)
            opsr["sddmm_u_add_v"] = op_record(
                "c2.sddmm_u_add_v", lambda: ops.gsddmm_u_add_v_mul_alpha(el, er, 1, g),
                4 * (N + 1) + E * (4 + H * b + 4 * H) + N * H * b, reps=50,
                gather=(N * H * b, E * H * b))
            opsr["segment_softmax"] = op_record(
                "c2.segment_softmax", lambda: ops.SegmentSoftmax(logits, 1, None, g),
                4 * (N + 1) + 8 * E * H, reps=50)
            opsr["spmm_u_mul_e"] = op_record(
                "c2.spmm_u_mul_e", lambda: ops.gspmm_src_mul_e_sum(z, att, [1], False, None, g),
                4 * (N + 1) + E * (4 + 4 * H + Fw * b) + N * Fw * b, reps=50, gather=rows)
            opsr["spmm_copy_u"] = op_record(
                "c2.spmm_copy_u", lambda: ops.SpMMSrc(z, [1], False, None, g),
                4 * (N + 1) + E * (4 + Fw * b) + N * Fw * b, reps=50, gather=rows)
        rec["ops"] = opsr = kept(opsr)
        if args.gather_ceiling and not only:
            rec["u_add_v_reference"] = u_add_v_reference(g, el.float().contiguous(), er.float().contiguous(), wl.src)
            rec["softmax_reference"] = softmax_reference(g, H)
        if "gat_aggregate" in opsr:
            rec["roofline"] = dict(opsr["gat_aggregate"],
                                   kernel="gat_aggregate (runs_kernel<GatPolicy<float, 4>> + fix-up)")
        if headline == "c2" and not args.no_cpu_baseline:
            import oracle
            ptr = g.in_pointer.cpu().numpy()
            nbr = g.in_node_indices.cpu().numpy()
            xt, wt = torch.from_numpy(x_h), torch.from_numpy(w_h)

            def cpu_layer():
                zc = torch.mm(xt, wt).numpy()
                zh = zc.reshape(N, H, -1)
                elc = (zh * a_h[0]).sum(-1).astype(np.float32)
                erc = (zh * a_h[1]).sum(-1).astype(np.float32)
                lg_ = oracle.sddmm_u_add_v(wl.src, wl.dst, elc, erc)
                lg_ = np.where(lg_ >= 0, lg_, np.float32(slope) * lg_).astype(np.float32)
                at = oracle.segment_softmax(ptr, None, lg_, zero_floor=True)
                return oracle.spmm_sum_f32(ptr, nbr, None, zc, at, op="u_mul_e", heads=H)

            cpu_ms, reps, ref = cpu_time(cpu_layer)
            got = out.cpu().numpy().reshape(ref.shape)
            cpu = {"value": round(E / (cpu_ms * 1e-3), 1), "unit": "edges/s",
                   "cores": oracle.num_threads(), "kind": "port", "ms_per_layer": round(cpu_ms, 2),
                   "sample": f"the full layer (all {E} edges), {reps} repetitions of the fp32 C port "
                             "(OpenMP) + torch-CPU dense projection",
                   "max_rel_diff_vs_gpu": float(np.abs(got - ref).max() / np.abs(ref).max())}
        return rec

    # ------------------------------------------------------------------ c3 ----
    def run_c3():
        wl = datasets.rgcn_zipf()                           # configs[2], seed 2
        N, E, R = wl.num_nodes, wl.num_edges, wl.num_etypes
        g = prepare_graph(wl.src, wl.dst, N, device=dev, etype_of=wl.etype, num_etypes=R)
        g.in_row_of_slot
        deg = torch.diff(g.in_pointer).clamp(min=1).float()
        norm = (1.0 / deg)[g.COO_dst].reshape(E, 1).contiguous()
        rec = {"workload": "configs[2]: 2-layer RGCN 16->64->8, 60 relations ~ Zipf(1.1), edges sorted "
                           "by type, right-normalised sum; uniform endpoints, seed 2",
               "num_nodes": N, "num_edges": E, "variants": {}}
        rng = np.random.default_rng(2)
        x_h = rng.standard_normal((N, 16), dtype=np.float32)
        w1_h, w2_h = datasets.glorot(rng, (R, 16, 64)), datasets.glorot(rng, (R, 64, 8))
        for dt, b, tag in ((torch.float32, 4, "f32"), (torch.bfloat16, 2, "bf16")):
            x, w1, w2 = (torch.from_numpy(t).to(dev).to(dt) for t in (x_h, w1_h, w2_h))

            def network():
                h1 = layers.rgcn_layer(g, x, w1, norm, fused=True, activation="relu")
                return layers.rgcn_layer(g, h1, w2, norm, fused=True)

            ms_step, _ = wall_time(network, max(args.steps, 100), max(args.warmup, 10),
                                   key=f"c3.step_{tag}")
            v = {"dtype": tag, "ms_per_step": r4(ms_step), "ms_per_layer": r4(ms_step, 2),
                 "edges_per_s": per_s(2 * E, ms_step), "ops": {}}
            h1 = torch.relu(layers.rgcn_layer(g, x, w1, norm, fused=True))
            for (K, M), xin, w in (((16, 64), x, w1), ((64, 8), h1, w2)):
                lbytes = 4 * (N + 1) + E * (8 + 4 + 4 + K * b) + R * K * M * b + N * M * b
                rows = (N * K * b, E * K * b)
                v["ops"][f"rgcn_layer_{K}_{M}"] = op_record(
                    f"c3.rgcn_layer_{K}_{M}_{tag}", lambda: layers.rgcn_layer(g, xin, w, norm, fused=True),
                    lbytes, 2.0 * E * K * M, tag, reps=50, gather=rows)
                # the same layer by its two implementations: the operator pair over an
                # (E, M) message tensor, and the single pass over destination tiles
                v["ops"][f"rgcn_layer_{K}_{M}_two_pass"] = op_record(
                    f"c3.rgcn_layer_{K}_{M}_two_pass_{tag}",
                    lambda: layers.rgcn_layer(g, xin, w, norm, fused="pair"),
                    lbytes + 2 * E * M * b, 2.0 * E * K * M, tag, reps=50, gather=rows)
                v["ops"][f"rgcn_layer_{K}_{M}_tiles"] = op_record(
                    f"c3.rgcn_layer_{K}_{M}_tiles_{tag}",
                    lambda: layers.rgcn_layer(g, xin, w, norm, fused="tiles"),
                    lbytes, 2.0 * E * K * M, tag, reps=50, gather=rows)
                if args.no_ops:
                    continue
                v["ops"][f"segment_mm_gather_{K}_{M}"] = op_record(
                    f"c3.segment_mm_gather_{K}_{M}_{tag}",
                    lambda: ops.SegmentMMEdgeGather(xin, w, 0, g, row_scale=norm),
                    E * (8 + 4 + (K + M) * b) + R * K * M * b, 2.0 * E * K * M, tag, reps=50,
                    gather=rows)
                xe = rnd(E, K, dtype=dt)
                v["ops"][f"segment_mm_edge_{K}_{M}"] = op_record(
                    f"c3.segment_mm_edge_{K}_{M}_{tag}", lambda: ops.SegmentMMEdge(xe, w, g),
                    E * (K + M) * b + R * K * M * b, 2.0 * E * K * M, tag, reps=50)
                m = rnd(E, M, dtype=dt)
                v["ops"][f"spmm_copy_e_{M}"] = op_record(
                    f"c3.spmm_copy_e_{M}_{tag}", lambda: ops.SpMMEdge(m, [1], False, None, g),
                    4 * (N + 1) + E * (4 + 4 + M * b) + N * M * b, reps=50)
            v["ops"] = kept(v["ops"])
            rec["variants"][tag] = v
        dom = rec["variants"]["f32"]["ops"].get("rgcn_layer_16_64")
        if dom is not None:
            rec["roofline"] = dict(dom, kernel="rgcn_layer 16->64 fp32 (one pass over destination tiles: "
                                               "typed product and neighbour sum on the matrix cores)")
        return rec

    # ------------------------------------------------------------------ c4 ----
    def run_c4():
        wl = datasets.hgt_hetero()                          # configs[3], seed 3
        N, E = wl.num_nodes, wl.num_edges
        Tn, Te = wl.num_ntypes, wl.num_etypes
        g = prepare_graph(wl.src, wl.dst, N, device=dev, ntype_of=wl.ntype, num_ntypes=Tn,
                          etype_of=wl.etype, num_etypes=Te)
        g.in_row_of_slot
        dt, b, H, D = torch.bfloat16, 2, 8, 16
        hid = H * D
        rng = np.random.default_rng(3)
        X = torch.from_numpy(rng.standard_normal((N, hid), dtype=np.float32)).to(dev).to(dt)
        wk, wq, wv, wa = (torch.from_numpy(datasets.glorot(rng, (Tn, hid, hid))).to(dev).to(dt)
                          for _ in range(4))
        ra, rm = (torch.from_numpy(datasets.glorot(rng, (Te, H, D, D))).to(dev).to(dt) for _ in range(2))
        rp = torch.from_numpy(datasets.glorot(rng, (Te, H), fan_in=H, fan_out=1)).to(dev).to(dt)
        skip = torch.ones(Tn, device=dev)

        def layer():
            return layers.hgt_layer(g, X, wk, wq, wv, wa, ra, rm, rp, skip, H, fused=True)

        ms_step, _ = wall_time(layer, max(args.steps, 50), max(args.warmup, 5), key="c4.step")
        rec = {"workload": "configs[3]: 1-layer HGT, 4 node types 40k/30k/20k/10k, 10 edge types, 8 heads "
                           "x 16, hidden 128, bf16 with fp32 accumulation; power-law out-degree, seed 3",
               "num_nodes": N, "num_edges": E, "dtype": "bf16",
               "ms_per_step": r4(ms_step), "edges_per_s": per_s(E, ms_step)}
        rows = N * hid * b                   # one (N, 128) bf16 table: 25.6 MB
        # bytes of the layer with its relation products per edge: h in, K/V/Q/t/out node rows,
        # three gathered rows per edge, the transformed values written and read once, scores
        # written and read once
        edges_bytes = N * hid * b * 9 + E * (3 * hid * b + 2 * hid * b + 24 + 4 * 4 * H)
        edges_flops = 2.0 * N * hid * hid * 4 + 4.0 * E * H * D * D
        # ... per (destination, relation) pair, the form the layer takes on this graph: node
        # rows as before, per edge the gathered k / v rows, the pair's transformed q row and
        # three index reads (scores stay in registers); per pair the q row read, its transform
        # written, the weighted sum and its transform written and read, the log-sum-exp
        # written, normalised in place and read
        P = g.relation_pairs().num_pairs
        pairs_bytes = N * hid * b * 9 + P * (hid * b * 6 + 4 * 4 * H) + E * (3 * hid * b + 12)
        pairs_flops = 2.0 * N * hid * hid * 4 + 4.0 * P * H * D * D + 4.0 * E * hid
        by_pairs = E >= layers.PAIRS_MIN_EDGES_PER_PAIR * P
        rec["num_pairs"] = P
        rec["relation_products"] = "per (destination, relation) pair" if by_pairs else "per edge"
        opsr = {"hgt_layer": op_record("c4.hgt_layer", layer, pairs_bytes if by_pairs else edges_bytes,
                                       pairs_flops if by_pairs else edges_flops, "bf16",
                                       gather=(3 * rows, E * 3 * hid * b))}
        if not args.no_ops:
            opsr["hgt_layer_per_edge"] = op_record(
                "c4.hgt_layer_per_edge",
                lambda: layers.hgt_layer(g, X, wk, wq, wv, wa, ra, rm, rp, skip, H, fused="edges"),
                edges_bytes, edges_flops, "bf16", gather=(3 * rows, E * 3 * hid * b))
            kk, vv, qq = ops.SegmentMMNodeStacked(X, [wk, wv, wq], g)
            opsr["relation_pair_attention"] = op_record(
                "c4.relation_pair_attention",
                lambda: ops.relation_pair_attention(kk, qq, vv, ra, rm, rp.float(), g,
                                                    factor=1.0 / D ** 0.5),
                pairs_bytes - N * hid * b * 6, pairs_flops - 2.0 * N * hid * hid * 4, "bf16",
                gather=(3 * rows, E * 3 * hid * b))
            opsr["segment_mm_node_128_128"] = op_record(
                "c4.segment_mm_node", lambda: ops.SegmentMMNode(X, wk, g),
                N * 2 * hid * b + Tn * hid * hid * b, 2.0 * N * hid * hid, "bf16", reps=50)
            wq, wv = rnd(Tn, hid, hid, dtype=dt) / hid ** 0.5, rnd(Tn, hid, hid, dtype=dt) / hid ** 0.5
            opsr["segment_mm_node_qkv_128_3x128"] = op_record(
                "c4.segment_mm_node_qkv", lambda: ops.SegmentMMNodeStacked(X, [wk, wq, wv], g),
                N * 4 * hid * b + 3 * Tn * hid * hid * b, 3 * 2.0 * N * hid * hid, "bf16", reps=50)
            opsr["segment_mm_dot_8x16x16"] = op_record(
                "c4.segment_mm_dot", lambda: ops.SegmentMMEdgeDot(X, ra, 0, X, 1, g),
                E * (16 + 2 * hid * b + 4 * H) + Te * H * D * D * b, 2.0 * E * H * D * D, "bf16", reps=50,
                gather=(rows, E * 2 * hid * b))
            opsr["segment_mm_gather_8x16x16"] = op_record(
                "c4.segment_mm_gather", lambda: ops.SegmentMMEdgeGather(X, rm, 0, g),
                E * (8 + 2 * hid * b) + Te * H * D * D * b, 2.0 * E * H * D * D, "bf16", reps=50,
                gather=(rows, E * hid * b))
            q, k = rnd(N, H, D, dtype=dt), rnd(N, H, D, dtype=dt)
            opsr["sddmm_u_dot_v"] = op_record(
                "c4.sddmm_u_dot_v", lambda: ops.gsddmm_u_dot_v(k, q, g),
                4 * (N + 1) + E * (4 + 2 * H * D * b + 4 * H), reps=50, gather=(2 * rows, E * 2 * hid * b))
            lg = rnd(E, H)
            opsr["segment_softmax"] = op_record(
                "c4.segment_softmax", lambda: ops.SegmentSoftmax(lg, 1, None, g),
                4 * (N + 1) + 8 * E * H, reps=50)
            att, v = torch.rand(E, H, device=dev), rnd(N, hid, dtype=dt)
            opsr["spmm_u_mul_e"] = op_record(
                "c4.spmm_u_mul_e", lambda: ops.gspmm_src_mul_e_sum(v, att, [1], False, None, g),
                4 * (N + 1) + E * (4 + 4 * H + hid * b) + N * hid * b, reps=50, gather=(rows, E * hid * b))
            ve = rnd(E, hid, dtype=dt)
            opsr["edge_softmax_sum"] = op_record(
                "c4.edge_softmax_sum", lambda: ops.edge_softmax_sum(lg, ve, g),
                4 * (N + 1) + E * (4 + 4 + 4 * H + hid * b) + N * hid * b, reps=50)
        rec["ops"] = opsr = kept(opsr)
        if "hgt_layer" in opsr:
            rec["roofline"] = dict(opsr["hgt_layer"], kernel="hgt_layer (3 node projections, relation "
                                   "products " + rec["relation_products"] + ", dot-product scores, edge "
                                   "softmax, weighted sum of gathered values, output projection)")
        if "segment_mm_node_qkv_128_3x128" in opsr:
            rec["mfma"] = dict(opsr["segment_mm_node_qkv_128_3x128"], kernel="K | Q | V projections 128 -> "
                               "3 x 128 bf16 (wide_mm_kernel, v_mfma_f32_16x16x32_bf16)")
        return rec

    # ------------------------------------------------------------------ c1 ----
    def run_c1():
        """configs[0]: the configuration the list assigns to the host cores (the reference's
        DGL CPU path, examples/GCN/GCN_DGL.py:11-14; DGL is not installed, so the host leg is
        the C port of SpMMSrc + torch-CPU products) with the same network on the GPU beside it."""
        nonlocal cpu
        wl = datasets.gcn_uniform()                         # seed 0
        N, E = wl.num_nodes, wl.num_edges
        g = prepare_graph(wl.src, wl.dst, N, device=dev)
        g.in_row_of_slot
        rng = np.random.default_rng(0)
        x_h = rng.standard_normal((N, 500), dtype=np.float32)
        w1_h, w2_h = datasets.glorot(rng, (500, 16)), datasets.glorot(rng, (16, 3))
        deg = np.bincount(wl.dst, minlength=N).astype(np.float32)     # in-degree, self loop included
        norm_h = (1.0 / np.sqrt(deg)).astype(np.float32)[:, None]     # symmetric normalisation
        x, w1, w2, norm = (torch.from_numpy(t).to(dev) for t in (x_h, w1_h, w2_h, norm_h))

        def network():
            h1 = layers.gcn_layer(g, x, w1, norm, norm, relu=True)
            return layers.gcn_layer(g, h1, w2, norm, norm, relu=False)

        ms_step, out = wall_time(network, max(args.steps, 100), max(args.warmup, 10), key="c1.step")
        rec = {"workload": "configs[0]: 2-layer GCN 500->16->3 with ReLU, symmetric degree normalisation, "
                           "fp32; uniform random graph (seed 0) + self loops",
               "num_nodes": N, "num_edges": E, "dtype": "f32",
               "ms_per_step": r4(ms_step), "edges_per_s": per_s(2 * E, ms_step)}
        opsr = {}
        for F_ in (16, 3):
            m = rnd(N, F_)
            opsr[f"spmm_copy_u_{F_}"] = op_record(
                f"c1.spmm_copy_u_{F_}", lambda: ops.SpMMSrc(m, [1], False, None, g),
                4 * (N + 1) + E * (4 + F_ * 4) + N * F_ * 4, reps=100, gather=(N * F_ * 4, E * F_ * 4))
        opsr["linear_500_16"] = op_record(
            "c1.linear_500_16", lambda: ops.linear(x, w1), 4 * (N * 500 + 500 * 16 + N * 16), reps=100)
        rec["ops"] = opsr = kept(opsr)
        if "spmm_copy_u_16" in opsr:
            rec["roofline"] = dict(opsr["spmm_copy_u_16"],
                                   kernel="SpMMSrc copy_u sum, F = 16 (runs_kernel<SpmmPolicy<float, 4>> + fix-up)")
        if not args.no_cpu_baseline:
            import oracle
            ptr = g.in_pointer.cpu().numpy()
            nbr = g.in_node_indices.cpu().numpy()
            xt, w1t, w2t, nt = (torch.from_numpy(t) for t in (x_h, w1_h, w2_h, norm_h))

            def cpu_network():
                m1 = (torch.mm(xt, w1t) * nt).numpy()
                h1 = torch.relu(torch.from_numpy(oracle.spmm_sum_f32(ptr, nbr, None, m1, op="copy_u")) * nt)
                m2 = (torch.mm(h1, w2t) * nt).numpy()
                return oracle.spmm_sum_f32(ptr, nbr, None, m2, op="copy_u") * norm_h

            cpu_ms, reps, ref = cpu_time(cpu_network, budget_s=3.0, min_reps=5, max_reps=200)
            got = out.cpu().numpy()
            host = {"value": round(2 * E / (cpu_ms * 1e-3), 1), "unit": "edges/s",
                    "cores": oracle.num_threads(), "torch_threads": torch.get_num_threads(),
                    "kind": "port", "ms_per_step": round(cpu_ms, 3), "passes": reps,
                    "sample": f"the whole 2-layer network (2 x {E} edges): one warm-up pass, then the mean "
                              f"of {reps} passes of the fp32 C port of SpMMSrc (OpenMP) + torch-CPU products",
                    "max_rel_diff_vs_gpu": float(np.abs(got - ref).max() / np.abs(ref).max())}
            rec["host_cores"] = host
            if ms_step is not None:
                rec["host_ms_over_gpu_ms"] = round(cpu_ms / ms_step, 1)
            if headline == "c1":
                cpu = host
        return rec

    runners = {"c1": run_c1, "c2": run_c2, "c3": run_c3, "c4": run_c4, "c5": run_c5}
    for c in wanted:
        results[c] = runners[c]()
        torch.cuda.empty_cache()
    # after the configurations, not before: where the caching allocator places a workload's
    # tensors changes the speed of the gather kernels (2 GiB allocated and released before
    # configs[4] is built made its step 11 % slower on every box tried), so each
    # configuration starts from an empty allocator and nothing is allocated ahead of it
    measured_copy = None if only else copy_rate()

    extra = {"profile_segments": segments} if args.markers else {}
    if only:                    # a profiler run: the operators asked for, nothing else
        print(json.dumps(dict({"only": sorted(only), "configs": results}, **extra)))
        return

    head = results[headline]
    if headline == "c3":
        hv = head["variants"]["f32"]
        ms_step, eps, dtype = hv["ms_per_step"], hv["edges_per_s"], "f32"
    else:
        ms_step, eps, dtype = head["ms_per_step"], head["edges_per_s"], head["dtype"]
    roof = head["roofline"]
    by_traffic = bool(roof.get("cache_served")) and roof.get("traffic") is not None
    roofline = {"kernel": roof["kernel"], "bound": "hbm",
                "achieved": round(roof["frac"] * HBM_PEAK_GBS, 1) if by_traffic else roof["effective_GBps"],
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": roof["frac"],
                "frac_basis": roof.get("frac_basis"),
                "traffic": roof.get("traffic"),
                "traffic_source": "profiles/hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE over the "
                                  "operator's own dispatches, separate runs; not measured in this run)",
                "algorithmic_bytes": roof["algorithmic_bytes"], "launch_ms": roof["ms"],
                "effective_GBps": roof["effective_GBps"],
                "cache_served": bool(roof.get("cache_served", False)),
                "peak_measured_copy_GBps": measured_copy}
    # the matrix-core figure the metric names: the best-placed MFMA kernel of the headline
    # configuration (else of any configuration measured in this run)
    mf = head.get("mfma") or next((results[c]["mfma"] for c in wanted if "mfma" in results[c]), None)
    if mf is not None:
        roofline["mfma"] = {"kernel": mf["kernel"], "tflops": mf["mfma_tflops"],
                            "peak_tflops": mf["mfma_peak_tflops"], "util": mf["mfma_util"],
                            "ceiling_tflops": mf["ceiling_tflops"],
                            "frac_of_ceiling": mf["frac_of_ceiling"],
                            "ceiling": "min(dense bf16 MFMA peak, arithmetic intensity x 8 TB/s)",
                            "launch_ms": mf["ms"]}
    metric = {"c1": "GCN", "c2": "GAT", "c5": "GAT", "c3": "RGCN", "c4": "HGT"}[headline]
    line = {
        "metric": metric + " layer fwd edges/s",
        "value": eps, "unit": "edges/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": head["workload"], "num_nodes": head["num_nodes"],
                   "num_edges": head["num_edges"]},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "peak_measured_copy_GBps": measured_copy,
        "configs": results,
    }
    line.update(extra)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
