"""Bench / report harness: log layout and table text of the reference's
python/graphiler/utils/bench.py:52-57 and artifact/plot.py:88-96 (CPU), and the
example networks under every execution mode (GPU)."""
import numpy as np
import pandas as pd
import pytest
import torch

from graphiler_amd import report


def test_log_layout_and_table(tmp_path):
    tags = ["0-DGL-UDF", "3-Graphiler"]
    logs = {}
    for i, name in enumerate(["cora", "reddit"]):
        log = report.init_log(tags, ["time", "mem"])
        assert list(log.index.names) == ["tag", "metric"] and log.shape == (4,)
        assert (log == 0).all()
        report.mark_unavailable(log, "0-DGL-UDF")
        log.at[("3-Graphiler", "time")] = 1.5 + i
        log.at[("3-Graphiler", "mem")] = 10.0 * (i + 1)
        logs[name] = log
    path = report.save_logs(logs, "GAT", str(tmp_path))
    frame = pd.read_pickle(path)            # written by this test a moment ago
    assert list(frame.columns) == ["cora", "reddit"]
    assert frame["reddit"][("3-Graphiler", "time")] == 2.5
    lines = (tmp_path / "GAT_time.dat").read_text().splitlines()
    assert lines[0].split("\t") == ["Dataset"] + tags
    assert lines[1].split("\t") == ["cora", "-1.0", "1.5"]
    assert lines[2].split("\t") == ["reddit", "-1.0", "2.5"]
    assert (tmp_path / "GAT_mem.dat").read_text().splitlines()[2].split("\t")[2] == "20.0"


def test_check_equal_tolerance():
    a = torch.tensor([1.0, 2.0, 3.0])
    assert report.check_equal(a, a * (1 + 5e-4))
    with pytest.raises(AssertionError):
        report.check_equal(a, a * (1 + 5e-3))
    assert report.check_equal(None, a) is False     # out-of-memory run: notice only


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["GCN", "GAT", "RGCN", "HGT"])
def test_example_networks_agree_across_modes(device, model, monkeypatch):
    """Two-layer network of each example model: the compiled plan at levels
    0 / 1 / 2 gives the eager PyTorch result (the reference's own check,
    bench.py:10-16, rtol 1e-3), and ``bench`` fills the log."""
    from graphiler_amd.examples import run
    monkeypatch.setitem(run.homo_dataset, "tiny", (24, 300, 2500, 9))
    monkeypatch.setitem(run.hetero_dataset, "tiny_kg", (300, 2500, 3, 5))
    dim = 24 if model in ("GCN", "GAT") else 16
    g, feats = run.load_data("tiny" if model in ("GCN", "GAT") else "tiny_kg", dim, device)
    net, extra = run._build(model, g, dim, device)
    log = report.init_log(["eager", "l0", "l1", "l2"], ["time", "mem"])
    with torch.no_grad():
        base = report.bench(net, (g, feats) + extra + ("eager",), tag="eager", repeat=2,
                            memory=True, log=log)
        assert base is not None and torch.isfinite(base).all() and float(base.abs().max()) > 0
        assert report.check_equal(net(g, feats, *extra, "eager64"), base)
        for level in (0, 1, 2):
            res = report.bench(net, (g, feats) + extra + (level,), tag=f"l{level}", repeat=2,
                               memory=True, log=log)
            assert report.check_equal(res, base)
    assert (log.xs("time", level="metric") > 0).all()


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["GAT", "HGT", "RGCN", "GCN"])
def test_network_replayed_as_hip_graph(device, model, monkeypatch):
    """A level-2 network recorded into a HIP graph: several replays, with new
    inputs written in place and eager work and synchronisations between them,
    each equal to the eager result on the same input."""
    from graphiler_amd.examples import run
    from graphiler_amd.hipgraph import Graphed
    monkeypatch.setitem(run.homo_dataset, "tiny", (24, 300, 2500, 9))
    monkeypatch.setitem(run.hetero_dataset, "tiny_kg", (300, 2500, 3, 5))
    dim = 24 if model in ("GCN", "GAT") else 16
    g, feats = run.load_data("tiny" if model in ("GCN", "GAT") else "tiny_kg", dim, device)
    net, extra = run._build(model, g, dim, device)
    with torch.no_grad():
        graphed = Graphed(net, (g, feats) + extra + (2,))
        for i in range(4):
            feats.copy_(torch.rand_like(feats) * (i + 1))
            want = net(g, feats, *extra, 2).clone()          # eager, same input
            torch.cuda.synchronize()
            got = graphed()
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"replay {i} differs from the eager run"
            net(g, torch.rand_like(feats), *extra, 0)        # unrelated eager work in between
