"""ga_gat_aggregate_static: the fused GAT aggregation with the library's own static
scratch buffer in place of a caller workspace, for callers that cannot allocate.

Called through the C ABI and compared bit for bit with ga_gat_aggregate (same kernels,
same order of every floating-point operation) on two calls in a row, the second on a
smaller graph, so that whatever the first call left in the shared buffer is there when
the second runs.  Runs last in the suite (file name) and also alone in a fresh
process, where its first call is the one that looks up the buffer's address.
"""
import numpy as np
import pytest
import torch

from graphiler_amd import capi, datasets, prepare_graph

pytestmark = pytest.mark.gpu


def _call(entry, g, el, er, z, out, heads, slope, ws=None):
    lib = capi.load()
    feat = z.shape[1]
    dt = capi.GA_F32 if z.dtype == torch.float32 else capi.GA_BF16
    stream = torch.cuda.current_stream(z.device).cuda_stream
    head = (g.in_pointer.data_ptr(), g.in_row_of_slot.data_ptr(), g.in_node_indices.data_ptr(),
            el.data_ptr(), er.data_ptr(), z.data_ptr(), out.data_ptr(), g.num_nodes,
            g.num_edges, heads, feat // heads, slope, dt)
    if entry == "static":
        rc = lib.ga_gat_aggregate_static(*head, stream)
    else:
        rc = lib.ga_gat_aggregate(*head, ws.data_ptr(), ws.numel(), stream)
    torch.cuda.synchronize()
    return rc


def _inputs(seed, n, feat, heads, dtype, device):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    z = torch.randn(n, feat, generator=gen).to(device).to(dtype)
    el = (torch.randn(n, heads, generator=gen) * 2).to(device)
    er = (torch.randn(n, heads, generator=gen) * 2).to(device)
    return el, er, z


@pytest.mark.parametrize("feat,heads,dtype", [(64, 1, torch.float32), (256, 4, torch.bfloat16),
                                              (17, 1, torch.float32)])
def test_static_scratch_matches_workspace_entry_point(device, feat, heads, dtype):
    lib = capi.load()
    # first a power-law graph whose hub rows span many workgroups, then a smaller one
    shapes = [dict(num_nodes=20_000, n_edges=1_500_000, scale=15, seed=3),
              dict(num_nodes=3_000, n_edges=40_000, scale=12, seed=4)]
    for i, shape in enumerate(shapes):
        wl = datasets.gat_rmat(**shape)
        g = prepare_graph(wl.src, wl.dst, wl.num_nodes, device=device)
        el, er, z = _inputs(10 + i, wl.num_nodes, feat, heads, dtype, device)
        ws = torch.empty(max(lib.ga_gat_workspace_bytes(g.num_edges, feat, heads), 256),
                         dtype=torch.uint8, device=device)
        want, got = torch.full_like(z, float("nan")), torch.full_like(z, float("nan"))
        assert _call("workspace", g, el, er, z, want, heads, 0.2, ws) == capi.GA_OK
        if i > 0:     # the first call on a device looks the buffer up; later ones do nothing else
            free_before = torch.cuda.mem_get_info(device)[0]
        rc_s = _call("static", g, el, er, z, got, heads, 0.2)
        assert rc_s == capi.GA_OK, lib.ga_error_string(rc_s)
        if i > 0:     # no device memory was taken from the driver
            assert torch.cuda.mem_get_info(device)[0] == free_before
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), \
            f"call {i}: static-scratch result differs from the workspace entry point"


def test_static_scratch_sizing_query_matches_the_entry_point(device):
    """ga_gat_static_scratch_needed (host arithmetic) says exactly when the entry point
    refuses: on real arrays, a width whose partial rows exceed the buffer gives
    GA_ESCRATCH with the output untouched, and the widest one that fits runs."""
    lib = capi.load()
    wl = datasets.gat_rmat(num_nodes=2_000, n_edges=1_200_000, scale=11, seed=5)
    g = prepare_graph(wl.src, wl.dst, wl.num_nodes, device=device)
    cap = 32 << 20
    heads = 3                       # several heads of an odd width: one feature per lane
    fits = [d for d in range(1, 4000, 2)
            if lib.ga_gat_static_scratch_needed(g.num_edges, heads, d, capi.GA_F32, 1) <= cap]
    assert fits and fits[-1] < 3999, "the sweep must cross the buffer's size"
    for dim, want in ((fits[-1], capi.GA_OK), (fits[-1] + 2, capi.GA_ESCRATCH)):
        el, er, z = _inputs(dim, wl.num_nodes, heads * dim, heads, torch.float32, device)
        out = torch.full_like(z, 7.0)
        rc = _call("static", g, el, er, z, out, heads, 0.2)
        assert rc == want, (dim, lib.ga_error_string(rc))
        if want == capi.GA_OK:
            ws = torch.empty(lib.ga_gat_workspace_bytes(g.num_edges, heads * dim, heads),
                             dtype=torch.uint8, device=device)
            ref = torch.empty_like(z)
            assert _call("workspace", g, el, er, z, ref, heads, 0.2, ws) == capi.GA_OK
            assert torch.equal(out, ref)
        else:
            assert b"static scratch" in lib.ga_error_string(rc)
            assert bool((out == 7.0).all())
