"""Wide bf16 typed products (csrc/wide_mm.hip): several weight tensors applied to the
same rows in one pass (ga_segment_mm_stacked, the K | Q | V projections of
examples/HGT/HGT.py:35-44) and the shapes of ga_segment_mm / ga_project_attn that the
same kernel takes (whole groups of 128 output columns; K % 8 == 0 up to 256, K % 4 == 0
up to 128).  Against
the oracle's segment_mm and a float64 product; the stacked form must give the bits of
separate calls."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from graphiler_amd import capi, datasets, ops
from helpers import TOL_BF16, TOL_F32, assert_close, to_bf16_f32

pytestmark = pytest.mark.gpu

COUNTS = [700, 0, 1, 333, 0, 64, 15, 129, 3000, 0, 257]      # rows per type, some empty


def _dev(a, device, bf16=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(device)
    return t.bfloat16() if bf16 else t


def _stacked(tp, X, Ws, M, dtype_code):
    lib = capi.load()
    rows, K = X.shape
    outs = [torch.full((rows, M), float("nan"), dtype=X.dtype, device=X.device) for _ in Ws]
    wp = (ctypes.c_void_p * len(Ws))(*[w.data_ptr() for w in Ws])
    yp = (ctypes.c_void_p * len(Ws))(*[o.data_ptr() for o in outs])
    rc = lib.ga_segment_mm_stacked(tp.data_ptr(), tp.numel() - 1, X.data_ptr(), wp, yp, len(Ws),
                                   rows, K, M, dtype_code, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    return outs


@pytest.mark.parametrize("K,M,n_w", [(128, 128, 3), (128, 128, 1), (128, 128, 4), (64, 128, 2),
                                     (32, 256, 2), (96, 128, 3), (160, 128, 2), (256, 128, 2),
                                     (256, 256, 1), (128, 256, 2), (64, 384, 1),
                                     # K % 32 != 0: padded fragments; K % 8 == 4: 8-byte row loads
                                     (40, 128, 3), (200, 128, 2), (100, 128, 2), (100, 256, 1),
                                     (36, 128, 1), (124, 256, 1)])
def test_stacked_products_wide(device, K, M, n_w):
    rng = np.random.default_rng(K + M + n_w)
    tp = np.concatenate([[0], np.cumsum(COUNTS)]).astype(np.int32)
    rows = int(tp[-1])
    X = to_bf16_f32(rng.standard_normal((rows, K), dtype=np.float32))
    Ws = [to_bf16_f32((rng.standard_normal((len(COUNTS), K, M)) / np.sqrt(K)).astype(np.float32))
          for _ in range(n_w)]
    dX, dtp = _dev(X, device, True), _dev(tp, device)
    dWs = [_dev(w, device, True) for w in Ws]
    outs = _stacked(dtp, dX, dWs, M, capi.GA_BF16)
    lib = capi.load()
    for w, dw, y in zip(Ws, dWs, outs):
        ref = oracle.segment_mm(tp, X, w)
        assert_close(y.float().cpu().numpy(), ref, TOL_BF16, f"stacked K={K} M={M} n={n_w}",
                     mag=oracle.segment_mm(tp, np.abs(X), np.abs(w)))
        one = torch.empty_like(y)
        assert lib.ga_segment_mm(dtp.data_ptr(), len(COUNTS), dX.data_ptr(), dw.data_ptr(),
                                 one.data_ptr(), rows, 1, K, M, capi.GA_BF16,
                                 torch.cuda.current_stream().cuda_stream) == 0
        assert torch.equal(one.view(torch.int16), y.view(torch.int16)), "stacked != separate calls"


@pytest.mark.parametrize("K,M,bf16", [(20, 24, False), (128, 128, False), (102, 128, True),
                                      (128, 64, True), (512, 128, True)])
def test_stacked_products_other_shapes(device, K, M, bf16):
    """Shapes outside the one-pass kernel run as one product per weight tensor."""
    rng = np.random.default_rng(K * 7 + M)
    counts = [70, 0, 333, 129]
    tp = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(tp[-1])
    X = rng.standard_normal((rows, K), dtype=np.float32)
    Ws = [(rng.standard_normal((len(counts), K, M)) / np.sqrt(K)).astype(np.float32) for _ in range(2)]
    if bf16:
        X, Ws = to_bf16_f32(X), [to_bf16_f32(w) for w in Ws]
    outs = _stacked(_dev(tp, device), _dev(X, device, bf16), [_dev(w, device, bf16) for w in Ws], M,
                    capi.GA_BF16 if bf16 else capi.GA_F32)
    for w, y in zip(Ws, outs):
        assert_close(y.float().cpu().numpy(), oracle.segment_mm(tp, X, w),
                     TOL_BF16 if bf16 else TOL_F32, f"stacked fallback K={K} M={M}")


def test_stacked_operator_and_hgt_projections(device):
    """ops.SegmentMMNodeStacked on a typed graph = three SegmentMMNode calls."""
    from graphiler_amd import prepare_graph
    rng = np.random.default_rng(8)
    n, e, tn = 900, 4000, 4
    ntype = np.sort(rng.integers(0, tn, n))
    src, dst = rng.integers(0, n, e), rng.integers(0, n, e)
    g = prepare_graph(src, dst, n, device=device, ntype_of=ntype, num_ntypes=tn)
    h = _dev(to_bf16_f32(rng.standard_normal((n, 128), dtype=np.float32)), device, True)
    ws = [_dev(to_bf16_f32(datasets.glorot(rng, (tn, 128, 128))), device, True) for _ in range(3)]
    outs = ops.SegmentMMNodeStacked(h, ws, g)
    for w, y in zip(ws, outs):
        assert torch.equal(ops.SegmentMMNode(h, w, g).view(torch.int16), y.view(torch.int16))
    with pytest.raises(RuntimeError):
        ops.SegmentMMNodeStacked(h, [ws[0], ws[1][:, :, :64].contiguous()], g)
    with pytest.raises(RuntimeError):
        ops.SegmentMMNodeStacked(h, [], g)


# shapes of the wide kernel, of the exact-shape tile kernel, and of the generic tile kernel
# (more than 8 column blocks or k blocks: fp32 M = 256 / 384, fp32 K = 256, bf16 K = 136 with
# three column groups), which takes no factor: the call must fall back, not drop it
FACTOR_SHAPES = [(128, 128, True), (256, 256, True), (100, 128, True), (64, 384, True),
                 (102, 128, True), (128, 64, True), (20, 24, False), (128, 128, False),
                 (16, 256, False), (32, 384, False), (256, 64, False), (136, 384, True),
                 (100, 384, True)]


@pytest.mark.parametrize("K,M,bf16", FACTOR_SHAPES)
def test_node_product_with_row_factor(device, K, M, bf16):
    """ops.SegmentMMNode(..., row_scale): the factor multiplies the fp32 sums (wide kernel,
    tile kernels, and shapes where it is applied afterwards)."""
    from graphiler_amd import prepare_graph
    rng = np.random.default_rng(K + M)
    tn = len(COUNTS)
    ntype = np.repeat(np.arange(tn), COUNTS)
    n = ntype.shape[0]
    src, dst = rng.integers(0, n, 2000), rng.integers(0, n, 2000)
    g = prepare_graph(src, dst, n, device=device, ntype_of=ntype, num_ntypes=tn)
    tp = np.concatenate([[0], np.cumsum(COUNTS)]).astype(np.int32)
    x = rng.standard_normal((n, K), dtype=np.float32)
    w = (rng.standard_normal((tn, K, M)) / np.sqrt(K)).astype(np.float32)
    if bf16:
        x, w = to_bf16_f32(x), to_bf16_f32(w)
    scale = rng.uniform(0.1, 2.0, n).astype(np.float32)
    got = ops.SegmentMMNode(_dev(x, device, bf16), _dev(w, device, bf16), g,
                            row_scale=_dev(scale, device).reshape(-1, 1))
    assert got.dtype == (torch.bfloat16 if bf16 else torch.float32) and got.shape == (n, M)
    ref = oracle.segment_mm(tp, x, w) * scale[:, None]
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 f"scaled node product K={K} M={M}",
                 mag=oracle.segment_mm(tp, np.abs(x), np.abs(w)) * scale[:, None])
    with pytest.raises(RuntimeError):
        ops.SegmentMMNode(_dev(x, device, bf16), _dev(w, device, bf16), g,
                          row_scale=_dev(scale[:-1], device))


@pytest.mark.parametrize("K,M,bf16", FACTOR_SHAPES)
@pytest.mark.parametrize("sigmoid", [True, False])
def test_node_product_with_type_gate(device, K, M, bf16, sigmoid):
    """ops.SegmentMMNodeGated: the per-node-type gate of an HGT layer's output projection
    (sigmoid(skip[ntype]), examples/HGT/HGT.py:58-60) applied inside the product where the
    wide kernel takes the shape, as a row factor elsewhere; against the oracle's product
    times the gate, and against the same gate handed over per row."""
    from graphiler_amd import prepare_graph
    rng = np.random.default_rng(K * 3 + M + int(sigmoid))
    tn = len(COUNTS)
    ntype = np.repeat(np.arange(tn), COUNTS)
    n = ntype.shape[0]
    src, dst = rng.integers(0, n, 2000), rng.integers(0, n, 2000)
    g = prepare_graph(src, dst, n, device=device, ntype_of=ntype, num_ntypes=tn)
    tp = np.concatenate([[0], np.cumsum(COUNTS)]).astype(np.int32)
    x = rng.standard_normal((n, K), dtype=np.float32)
    w = (rng.standard_normal((tn, K, M)) / np.sqrt(K)).astype(np.float32)
    if bf16:
        x, w = to_bf16_f32(x), to_bf16_f32(w)
    gate = rng.uniform(-3.0, 3.0, tn).astype(np.float32)
    factor = (1.0 / (1.0 + np.exp(-gate.astype(np.float64)))) if sigmoid else gate.astype(np.float64)
    got = ops.SegmentMMNodeGated(_dev(x, device, bf16), _dev(w, device, bf16), _dev(gate, device), g,
                                 sigmoid=sigmoid)
    assert got.dtype == (torch.bfloat16 if bf16 else torch.float32) and got.shape == (n, M)
    ref = oracle.segment_mm(tp, x, w) * factor[ntype][:, None]
    assert_close(got.float().cpu().numpy(), ref, TOL_BF16 if bf16 else TOL_F32,
                 f"gated node product K={K} M={M} sigmoid={sigmoid}",
                 mag=oracle.segment_mm(tp, np.abs(x), np.abs(w)) * np.abs(factor)[ntype][:, None])
    per_row = ops.SegmentMMNode(_dev(x, device, bf16), _dev(w, device, bf16), g,
                                row_scale=_dev(factor[ntype].astype(np.float32), device))
    # the two differ by the rounding of the factor only (fp32 sigmoid in the kernel)
    assert_close(got.float().cpu().numpy(), per_row.float().cpu().numpy(),
                 8e-3 if bf16 else TOL_F32, "gate inside the product against the gate per row")
    with pytest.raises(RuntimeError):
        ops.SegmentMMNodeGated(_dev(x, device, bf16), _dev(w, device, bf16), _dev(gate[:-1], device), g)


@pytest.mark.parametrize("rows,K,M,heads", [
    (1500, 256, 256, 4), (1500, 256, 256, 2), (1500, 256, 256, 8),   # heads of 64, 128, 32 columns
    (777, 128, 128, 1), (777, 128, 128, 4), (333, 64, 384, 3), (255, 32, 512, 8),
    (1, 96, 128, 2), (4097, 160, 256, 4),
    (3001, 100, 256, 4), (515, 36, 128, 2), (90, 248, 256, 4), (777, 124, 128, 4)])
def test_project_attn_wide(device, rows, K, M, heads):
    """The projection with attention terms at the widths of the one-pass kernel."""
    rng = np.random.default_rng(rows + K + M + heads)
    x = to_bf16_f32(rng.standard_normal((rows, K), dtype=np.float32))
    w = to_bf16_f32(datasets.glorot(rng, (K, M)))
    a = rng.standard_normal((2, heads, M // heads), dtype=np.float32)
    z, el, er = ops.linear_attn(_dev(x, device, True), _dev(w, device, True),
                                _dev(a[0], device), _dev(a[1], device))
    assert z.dtype == torch.bfloat16 and el.dtype == torch.float32 and el.shape == (rows, heads)
    zr = x.astype(np.float64) @ w.astype(np.float64)
    assert_close(z.float().cpu().numpy(), zr, TOL_BF16, "wide project z")
    zh = zr.reshape(rows, heads, -1)
    mag_l = (np.abs(zh) * np.abs(a[0])).sum(-1)
    mag_r = (np.abs(zh) * np.abs(a[1])).sum(-1)
    # el / er come from the fp32 accumulators, not from the rounded z
    assert_close(el.cpu().numpy(), (zh * a[0]).sum(-1), TOL_F32, "wide project el", mag=mag_l)
    assert_close(er.cpu().numpy(), (zh * a[1]).sum(-1), TOL_F32, "wide project er", mag=mag_r)


@pytest.mark.parametrize("seed", range(12))
def test_wide_products_random_shapes(device, seed):
    """Random row counts per type (empty types, a single row, types that end inside a
    step), type counts either side of the kernel's limit of 64, K from 4 to 256, one to
    four weights of 128 to 512 columns: whatever kernel a shape lands on, the result is
    the oracle's and the stacked call gives the bits of separate calls."""
    rng = np.random.default_rng(1000 + seed)
    n_types = int(rng.choice([1, 2, 5, 63, 64, 65, 130]))
    counts = rng.choice([0, 1, 7, 31, 128, 129, 300, 1000], size=n_types,
                        p=[.2, .1, .1, .1, .1, .1, .2, .1])
    if counts.sum() == 0:
        counts[0] = 5
    tp = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(tp[-1])
    K = int(rng.choice([4, 8, 20, 32, 36, 64, 100, 128, 192, 256]))
    M = int(rng.choice([128, 256, 384, 512]))
    n_w = int(rng.integers(1, 5))
    X = to_bf16_f32(rng.standard_normal((rows, K), dtype=np.float32))
    Ws = [to_bf16_f32((rng.standard_normal((n_types, K, M)) / np.sqrt(K)).astype(np.float32))
          for _ in range(n_w)]
    dX, dtp = _dev(X, device, True), _dev(tp, device)
    dWs = [_dev(w, device, True) for w in Ws]
    outs = _stacked(dtp, dX, dWs, M, capi.GA_BF16)
    lib = capi.load()
    for w, dw, y in zip(Ws, dWs, outs):
        assert_close(y.float().cpu().numpy(), oracle.segment_mm(tp, X, w), TOL_BF16,
                     f"random wide T={n_types} rows={rows} K={K} M={M} n={n_w}")
        one = torch.empty_like(y)
        assert lib.ga_segment_mm(dtp.data_ptr(), n_types, dX.data_ptr(), dw.data_ptr(),
                                 one.data_ptr(), rows, 1, K, M, capi.GA_BF16,
                                 torch.cuda.current_stream().cuda_stream) == 0
        assert torch.equal(one.view(torch.int16), y.view(torch.int16))
