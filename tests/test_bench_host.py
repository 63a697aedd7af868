"""Host-side pieces of the benchmark script: argument handling that needs no GPU and
the per-operator traffic table it reads from profiles/."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args],
                          capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0 and "ONE GPU" in r.stderr


def test_unknown_configuration_is_refused():
    r = _run("--configs", "c9")
    assert r.returncode != 0 and "unknown configuration" in r.stderr


def test_traffic_table_has_a_count_for_every_benchmarked_operator():
    import bench
    table = bench.load_traffic()
    # the operators every default run reports (keys of op_record / wall_time in bench.py)
    wanted = ["c5.step", "c5.gat_aggregate_from_z", "c5.gat_aggregate", "c5.spmm_u_mul_e",
              "c5.sddmm_u_add_v", "c5.segment_softmax", "c5.project_attn_100_256",
              "c5.project_attn_256_256", "c2.step", "c2.gat_aggregate", "c2.linear_attn",
              "c2.sddmm_u_add_v", "c2.segment_softmax", "c2.spmm_u_mul_e", "c2.spmm_copy_u",
              "c4.step", "c4.hgt_layer", "c4.hgt_layer_per_edge", "c4.relation_pair_attention",
              "c4.segment_mm_node", "c4.segment_mm_node_qkv", "c4.segment_mm_dot",
              "c4.segment_mm_gather", "c4.sddmm_u_dot_v", "c4.segment_softmax", "c4.spmm_u_mul_e",
              "c4.edge_softmax_sum", "c1.step", "c1.spmm_copy_u_16", "c1.spmm_copy_u_3",
              "c1.linear_500_16"]
    for tag in ("f32", "bf16"):
        wanted.append(f"c3.step_{tag}")
        for k, m in ((16, 64), (64, 8)):
            wanted += [f"c3.rgcn_layer_{k}_{m}_{tag}", f"c3.rgcn_layer_{k}_{m}_two_pass_{tag}",
                       f"c3.rgcn_layer_{k}_{m}_tiles_{tag}", f"c3.segment_mm_gather_{k}_{m}_{tag}",
                       f"c3.segment_mm_edge_{k}_{m}_{tag}", f"c3.spmm_copy_e_{m}_{tag}"]
    missing = [k for k in wanted if k not in table]
    assert not missing, missing
    assert all(v > 0 for v in table.values())
    # a count can only be an operator's own when it covers what the operator writes:
    # the per-edge product of config 4 writes 2 M rows of 256 bytes, the fused layer its
    # (N, 128) bf16 result and the tensors between its kernels
    assert table["c4.segment_mm_gather"] >= 2_000_000 * 256
    assert table["c4.hgt_layer"] >= 100_000 * 256
    assert table["c5.gat_aggregate_from_z"] >= 2_449_029 * 512
