"""The one-pass RGCN aggregation (ops.TypedSpMMEdge, ga_typed_tiles_build + ga_typed_spmm)
against the oracle's operator chain it replaces: gather_rows -> segment_mm -> * norm ->
spmm(copy_e), i.e. BroadcastSrcNode -> SegmentMMEdge -> mul -> SpMMEdge of
examples/RGCN/RGCN.py:25-33.  fp32 within 1e-5 (norm and element-wise against the sum
of the absolute messages), bf16 within 2e-2; identical bits from call to call; messages
that are not finite reach exactly the rows the chain gives them to."""
import numpy as np
import pytest
import torch

import oracle
from graphiler_amd import capi, layers, ops, prepare_graph
from graphiler_amd.graph import build_graph_arrays, sort_edges_by_type
from helpers import TOL_BF16, TOL_F32, assert_close, to_bf16_f32

pytestmark = pytest.mark.gpu


def _typed_graph(rng, n, e, r, device, hub=False):
    src = rng.integers(0, n, e, dtype=np.int64)
    dst = rng.integers(0, n, e, dtype=np.int64)
    if hub and e:
        dst[: e // 3] = n // 2          # one destination with a third of the edges
    p = np.arange(1, r + 1, dtype=np.float64) ** -1.1
    etype = rng.choice(r, size=e, p=p / p.sum()).astype(np.int64)
    src, dst, etype, _ = sort_edges_by_type(src, dst, etype)
    g = prepare_graph(src, dst, n, device=device, etype_of=etype, num_etypes=r)
    return g, build_graph_arrays(src, dst, n), src, dst, etype


def _dev(a, device, bf16=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(device)
    return t.bfloat16() if bf16 else t


def _reference(arr, src, etype, r, x, w, norm):
    """The operator chain on the oracle, and the magnitude its result is held against:
    the same chain on absolute values (every product of the typed product and every
    message of the sum counted with its size)."""
    etp = oracle.type_pointer(etype, r)
    args = (arr.in_pointer, arr.in_node_indices, arr.in_edge_indices)
    out = []
    for xx, ww in ((x, w), (np.abs(x), np.abs(w))):
        msg = oracle.segment_mm(etp, oracle.gather_rows(src, xx), ww)
        if norm is not None:
            msg = msg * norm[:, None]
        out.append(oracle.spmm(*args, msg.astype(np.float32), op="copy_e"))
    return out[0], out[1]


CASES = [  # nodes, edges, relations, K, M, hub
    (300, 4000, 7, 16, 64, False),
    (1000, 20000, 60, 16, 64, True),
    (130, 900, 3, 32, 64, False),
    (257, 5000, 11, 48, 64, True),
    (128, 3000, 5, 64, 64, False),
    (5, 40, 2, 16, 64, False),
    (700, 0, 4, 16, 64, False),
    # narrower outputs: one wavefront per chunk, four taking turns on a tile's chunks
    (1000, 20000, 60, 64, 8, True),
    (300, 4000, 7, 16, 8, False),
    (257, 5000, 11, 48, 16, True),
    (130, 900, 3, 32, 32, False),
    (1000, 20000, 60, 64, 32, True),
    (5, 40, 2, 64, 16, False),
    (700, 0, 4, 64, 8, False),
]


@pytest.mark.parametrize("n,e,r,k,m,hub", CASES)
@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
@pytest.mark.parametrize("scaled", [True, False], ids=["norm", "plain"])
def test_typed_spmm_matches_operator_chain(device, n, e, r, k, m, hub, bf16, scaled):
    rng = np.random.default_rng(n + e + k + m)
    g, arr, src, dst, etype = _typed_graph(rng, n, e, r, device, hub)
    x = rng.standard_normal((n, k), dtype=np.float32)
    w = (rng.standard_normal((r, k, m)) / np.sqrt(k)).astype(np.float32)
    norm = rng.uniform(0.1, 1.5, e).astype(np.float32) if scaled else None
    if bf16:
        x, w = to_bf16_f32(x), to_bf16_f32(w)
    got = ops.TypedSpMMEdge(_dev(x, device, bf16), _dev(w, device, bf16), g,
                            row_scale=_dev(norm, device) if scaled else None)
    assert got.shape == (n, m) and got.dtype == (torch.bfloat16 if bf16 else torch.float32)
    ref, mag = _reference(arr, src, etype, r, x, w, norm)
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 f"typed spmm n={n} e={e} r={r} k={k} m={m}", mag=mag)
    again = ops.TypedSpMMEdge(_dev(x, device, bf16), _dev(w, device, bf16), g,
                              row_scale=_dev(norm, device) if scaled else None)
    assert torch.equal(got.view(torch.int16 if bf16 else torch.int32),
                       again.view(torch.int16 if bf16 else torch.int32)), "bits differ between calls"


def test_typed_tiles_layout(device):
    """The prepared layout itself (integer work, exact): every edge appears once, in a
    chunk of its relation inside the tile of its destination; pad slots say -1 / 255;
    chunks of a tile are contiguous and ordered by relation, slots inside a (tile,
    relation) group by adjacency position."""
    rng = np.random.default_rng(9)
    n, e, r = 700, 9000, 13
    g, arr, src, dst, etype = _typed_graph(rng, n, e, r, device, hub=True)
    *arrays, rows = ops._typed_tiles(g)
    tcp, ctype, ssrc, sdst, sedge = (t.cpu().numpy() for t in arrays)
    assert rows in (128, 144) and rows == capi.load().ga_typed_tile_rows(n)
    tiles = -(-n // rows)
    assert tcp.shape == (tiles + 1,) and tcp[0] == 0 and np.all(np.diff(tcp) >= 0)
    total = int(tcp[-1])
    used = slice(0, 16 * total)
    live = sedge[used] >= 0
    assert np.array_equal(np.sort(sedge[used][live]), np.arange(e)), "every edge once"
    assert np.all(ssrc[used][~live] == -1) and np.all(sdst[used][~live] == 255)
    ed = sedge[used][live]
    assert np.array_equal(ssrc[used][live], src[ed])
    chunk_of_slot = np.arange(16 * total) // 16
    tile_of_chunk = np.searchsorted(tcp, np.arange(total), side="right") - 1
    assert np.array_equal(dst[ed], tile_of_chunk[chunk_of_slot[live]] * rows + sdst[used][live])
    assert np.array_equal(etype[ed], (ctype[:total] & 0xffff)[chunk_of_slot[live]])
    blocks = np.zeros(total, dtype=np.int64)          # 16-row blocks a chunk has rows in
    np.bitwise_or.at(blocks, chunk_of_slot[live], 1 << (sdst[used][live].astype(np.int64) >> 4))
    assert np.array_equal(ctype[:total].astype(np.int64) >> 16, blocks)
    # order: relation ascending inside a tile; a group's slots in adjacency order
    for t in range(tiles):
        ct = ctype[tcp[t]:tcp[t + 1]] & 0xffff
        assert np.all(np.diff(ct) >= 0)
    slot_of_edge = np.empty(e, dtype=np.int64)
    slot_of_edge[arr.in_edge_indices] = np.arange(e)
    pos = slot_of_edge[ed]
    key = tile_of_chunk[chunk_of_slot[live]] * r + etype[ed]
    same = key[1:] == key[:-1]
    assert np.all(pos[1:][same] > pos[:-1][same])
    # every group wastes less than one chunk
    groups = len(np.unique(key))
    assert total <= -(-e // 16) + groups
    assert total <= capi.load().ga_typed_tiles_chunk_capacity(n, e, r, rows)


@pytest.mark.parametrize("m", [64, 8, 32])
@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
def test_typed_spmm_messages_that_are_not_finite(device, bf16, m):
    """inf and NaN source features: the rows that receive such a message become what
    the chain makes them (inf, -inf or NaN), every other row stays finite and exact to
    tolerance -- the selection matrices of the kernel must not spread them."""
    rng = np.random.default_rng(31)
    n, e, r, k = 400, 6000, 6, 16
    g, arr, src, dst, etype = _typed_graph(rng, n, e, r, device)
    x = rng.standard_normal((n, k), dtype=np.float32)
    w = np.abs(rng.standard_normal((r, k, m)) / np.sqrt(k)).astype(np.float32) + 0.01
    if bf16:
        x, w = to_bf16_f32(x), to_bf16_f32(w)
    x[0, :] = np.inf            # +inf messages (weights are positive); row 0 is also what pad slots read
    x[77, :] = -np.inf
    x[200, 5] = np.nan
    norm = rng.uniform(0.1, 1.5, e).astype(np.float32)
    got = ops.TypedSpMMEdge(_dev(x, device, bf16), _dev(w, device, bf16), g,
                            row_scale=_dev(norm, device)).float().cpu().numpy()
    with np.errstate(invalid="ignore", over="ignore"):
        ref, _ = _reference(arr, src, etype, r, x, w, norm)
    touched = np.zeros(n, dtype=bool)
    touched[dst[np.isin(src, [0, 77, 200])]] = True
    assert touched.any() and not touched.all()
    assert np.all(np.isfinite(got[~touched])), "a row without such a message is not finite"
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(np.isposinf(got), np.isposinf(ref))
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))
    fin = np.isfinite(ref)
    tol = TOL_BF16 if bf16 else TOL_F32
    assert np.abs(got[fin] - ref[fin]).max() <= tol * np.abs(ref[fin]).max()


def test_rgcn_layer_paths_agree(device):
    rng = np.random.default_rng(4)
    n, e, r = 500, 8000, 9
    g, arr, src, dst, etype = _typed_graph(rng, n, e, r, device)
    x = _dev(rng.standard_normal((n, 16), dtype=np.float32), device)
    w = _dev((rng.standard_normal((r, 16, 64)) / 4).astype(np.float32), device)
    norm = _dev(rng.uniform(0.1, 1.0, (e, 1)).astype(np.float32), device)
    a = layers.rgcn_layer(g, x, w, norm, fused="tiles")
    b = layers.rgcn_layer(g, x, w, norm, fused=False)
    c = layers.rgcn_layer(g, x, w, norm, fused=True)
    d = layers.rgcn_layer(g, x, w, norm, fused="pair")
    assert_close(a.cpu().numpy(), b.cpu().numpy(), 2 * TOL_F32, "tiles against unfused")
    assert_close(c.cpu().numpy(), b.cpu().numpy(), 2 * TOL_F32, "default against unfused")
    assert_close(d.cpu().numpy(), b.cpu().numpy(), 2 * TOL_F32, "pair against unfused")
    assert torch.equal(a, c), "16 -> 64 takes the single pass by default"
    # a second layer as in the two-layer network (64 -> 8: single pass) and a wide one (pair)
    for k, m, one_pass in ((64, 8, True), (64, 64, False)):
        x2 = _dev(rng.standard_normal((n, k), dtype=np.float32), device)
        w2 = _dev((rng.standard_normal((r, k, m)) / 8).astype(np.float32), device)
        assert ops.typed_spmm_preferred(x2, w2) == one_pass
        got = layers.rgcn_layer(g, x2, w2, norm, fused=True)
        want = layers.rgcn_layer(g, x2, w2, norm, fused="tiles" if one_pass else "pair")
        assert torch.equal(got, want)
        assert_close(got.cpu().numpy(), layers.rgcn_layer(g, x2, w2, norm, fused=False).cpu().numpy(),
                     2 * TOL_F32, f"{k} -> {m} against unfused")


def test_rgcn_layer_on_a_hub_keeps_fp32_accuracy(device):
    """A destination with 60,000 in-edges whose messages all have one sign: the one-pass
    kernel adds them chunk after chunk into one accumulator and drifts with the in-degree,
    so the fp32 layer (and the TorchScript operator) must take the operator pair, whose
    run-wise sums hold the 1e-5 element by element; bf16 keeps the single pass."""
    from graphiler_amd import torch_boundary
    rng = np.random.default_rng(77)
    n, r, hub = 400, 5, 60_000
    e = hub + 3000
    src = rng.integers(0, n, e)
    dst = rng.integers(0, n, e)
    dst[:hub] = 11
    etype = rng.integers(0, r, e)
    src, dst, etype, _ = sort_edges_by_type(src, dst, etype)
    g = prepare_graph(src, dst, n, device=device, etype_of=etype, num_etypes=r)
    arr = build_graph_arrays(src, dst, n)
    assert g.max_in_degree >= hub > ops.TYPED_SPMM_MAX_IN_DEGREE_F32
    x = np.abs(rng.standard_normal((n, 16), dtype=np.float32))
    w = np.abs(rng.standard_normal((r, 16, 64)) / 4).astype(np.float32)
    norm = rng.uniform(0.5, 1.0, (e, 1)).astype(np.float32)
    etp = oracle.type_pointer(etype, r)
    msg = (oracle.segment_mm(etp, oracle.gather_rows(src, x), w) * norm).astype(np.float32)
    ref = oracle.spmm(arr.in_pointer, arr.in_node_indices, arr.in_edge_indices, msg, op="copy_e")
    dx, dw, dn = _dev(x, device), _dev(w, device), _dev(norm, device)
    assert not ops.typed_spmm_preferred(dx, dw, g) and ops.typed_spmm_preferred(dx, dw)
    got = layers.rgcn_layer(g, dx, dw, dn, fused=True)
    assert_close(got.cpu().numpy(), ref, TOL_F32, "fp32 RGCN layer with a 60,000-edge row", mag=ref)
    assert torch.equal(got, layers.rgcn_layer(g, dx, dw, dn, fused="pair"))
    torch_boundary.load()
    scripted = torch.ops.my_ops.TypedSpMMEdge(dx, dw, dn, torch_boundary.script_graph(g))
    assert_close(scripted.cpu().numpy(), ref, TOL_F32, "my_ops::TypedSpMMEdge with a 60,000-edge row",
                 mag=ref)
    # bf16 (2e-2): the single pass stays
    xb, wb = dx.bfloat16(), dw.bfloat16()
    assert ops.typed_spmm_preferred(xb, wb, g)
    assert torch.equal(layers.rgcn_layer(g, xb, wb, dn, fused=True),
                       layers.rgcn_layer(g, xb, wb, dn, fused="tiles"))


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
def test_typed_spmm_activation(device, bf16):
    """The activation applied to the fp32 sums inside the kernel against the same
    activation on the plain result (relu: exactly; elu: to rounding), for both column
    layouts, and through rgcn_layer for the one-pass and the two-pass form."""
    import torch.nn.functional as F
    rng = np.random.default_rng(15)
    n, e, r = 700, 9000, 8
    g, arr, src, dst, etype = _typed_graph(rng, n, e, r, device)
    norm = _dev(rng.uniform(0.1, 1.5, (e, 1)).astype(np.float32), device)
    for k, m in ((16, 64), (64, 8)):
        x = _dev(rng.standard_normal((n, k), dtype=np.float32), device, bf16)
        w = _dev((rng.standard_normal((r, k, m)) / np.sqrt(k)).astype(np.float32), device, bf16)
        plain = ops.TypedSpMMEdge(x, w, g, row_scale=norm.reshape(-1))
        relu = ops.TypedSpMMEdge(x, w, g, row_scale=norm.reshape(-1), activation="relu")
        assert torch.equal(relu, torch.relu(plain)) and bool((relu == 0).any())
        elu = ops.TypedSpMMEdge(x, w, g, row_scale=norm.reshape(-1), activation="elu")
        assert_close(elu.float().cpu().numpy(), F.elu(plain.float()).cpu().numpy(),
                     TOL_BF16 if bf16 else TOL_F32, f"typed elu {k}->{m}")
        if not bf16:
            # sums near 1e-4, element by element: expm1, not exp(o) - 1
            xs = x * 1e-4
            want = F.elu(ops.TypedSpMMEdge(xs, w, g, row_scale=norm.reshape(-1))).cpu().numpy()
            got = ops.TypedSpMMEdge(xs, w, g, row_scale=norm.reshape(-1), activation="elu")
            assert_close(got.cpu().numpy(), want, TOL_F32, f"typed elu near 1e-4 {k}->{m}",
                         mag=np.abs(want))
        for fused in ("tiles", "pair", False):
            got = layers.rgcn_layer(g, x, w, norm, fused=fused, activation="relu")
            want = torch.relu(layers.rgcn_layer(g, x, w, norm, fused=fused))
            assert torch.equal(got, want), fused
    with pytest.raises(RuntimeError):
        ops.TypedSpMMEdge(x, w, g, activation="tanh")
    with pytest.raises(RuntimeError):
        layers.rgcn_layer(g, x, w, norm, activation="tanh")


def test_typed_spmm_rejects_what_it_does_not_cover(device):
    rng = np.random.default_rng(6)
    g, arr, src, dst, etype = _typed_graph(rng, 100, 500, 3, device)
    x = torch.randn(100, 16, device=device)
    with pytest.raises(capi.GraphilerError):          # M not one of 8, 16, 32, 64
        ops.TypedSpMMEdge(x, torch.randn(3, 16, 24, device=device), g)
    with pytest.raises(capi.GraphilerError):
        ops.TypedSpMMEdge(x, torch.randn(3, 16, 128, device=device), g)
    with pytest.raises(capi.GraphilerError):          # K not a multiple of 16
        ops.TypedSpMMEdge(torch.randn(100, 8, device=device), torch.randn(3, 8, 64, device=device), g)
    with pytest.raises(RuntimeError):                 # one weight per relation
        ops.TypedSpMMEdge(x, torch.randn(4, 16, 64, device=device), g)
    with pytest.raises(RuntimeError):
        ops.TypedSpMMEdge(x, torch.randn(3, 16, 64, device=device).bfloat16(), g)
    with pytest.raises(RuntimeError):
        ops.TypedSpMMEdge(x.cpu(), torch.randn(3, 16, 64), g)
    assert not ops.typed_spmm_supported(x, torch.randn(3, 16, 24, device=device))
    assert ops.typed_spmm_supported(x, torch.randn(3, 16, 64, device=device))
    assert ops.typed_spmm_supported(x, torch.randn(3, 16, 8, device=device))


@pytest.mark.parametrize("seed", range(16))
def test_typed_spmm_random_graphs(device, seed):
    """Random sizes either side of a tile, relation counts from 1 to 200 (most of them
    without edges in most tiles), a destination that takes a large share of the edges,
    both dtypes, with and without the per-edge factor."""
    rng = np.random.default_rng(500 + seed)
    n = int(rng.choice([1, 17, 127, 128, 129, 144, 145, 1000, 5000]))
    e = int(rng.choice([0, 1, 50, 3000, 40000]))
    r = int(rng.choice([1, 2, 9, 60, 200]))
    k = int(rng.choice([16, 32, 64]))
    m = int(rng.choice([8, 16, 32, 64]))
    bf16 = bool(rng.integers(0, 2))
    scaled = bool(rng.integers(0, 2))
    g, arr, src, dst, etype = _typed_graph(rng, n, e, r, device, hub=bool(rng.integers(0, 2)))
    x = rng.standard_normal((n, k), dtype=np.float32)
    w = (rng.standard_normal((r, k, m)) / np.sqrt(k)).astype(np.float32)
    norm = rng.uniform(0.1, 1.5, e).astype(np.float32) if scaled else None
    if bf16:
        x, w = to_bf16_f32(x), to_bf16_f32(w)
    got = ops.TypedSpMMEdge(_dev(x, device, bf16), _dev(w, device, bf16), g,
                            row_scale=_dev(norm, device) if scaled else None)
    ref, mag = _reference(arr, src, etype, r, x, w, norm)
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 f"typed random n={n} e={e} r={r} k={k} m={m} bf16={bf16}", mag=mag)
