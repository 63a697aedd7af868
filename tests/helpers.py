"""Shared helpers for the parity tests."""
import os

import numpy as np

# Tolerances of the parity contract: fp32 device results within 1e-5 of the
# fp64-accumulated oracle, bf16 results within 2e-2 of the fp32 oracle, both
# relative to the magnitude of the reference output.
TOL_F32 = 1e-5
TOL_BF16 = 2e-2


def rel_err(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if ref.size == 0:
        return 0.0
    finite = np.isfinite(ref)
    assert np.array_equal(np.isfinite(got), finite), "non-finite pattern differs"
    assert np.array_equal(got[~finite], ref[~finite]), "infinities differ"
    scale = max(np.abs(ref[finite]).max(initial=0.0), 1e-30)
    return float(np.abs(got[finite] - ref[finite]).max(initial=0.0) / scale)


def elementwise_err(got, ref, mag):
    """max_i |got_i - ref_i| / mag_i, where mag_i >= |ref_i| is the magnitude the
    element is held against: the same expression evaluated on absolute values (the
    sum of the absolute terms of a reduction), or |ref_i| itself for an output that
    is not a sum of signed terms (softmax weights).  This is the per-element reading
    of "within 1e-5 relative": an output that is small because its terms cancel is
    held to the size of its terms, every other one to its own size."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    mag = np.abs(np.asarray(mag, dtype=np.float64))
    assert got.shape == ref.shape == mag.shape, (got.shape, ref.shape, mag.shape)
    if ref.size == 0:
        return 0.0
    finite = np.isfinite(ref)
    assert np.array_equal(np.isfinite(got), finite), "non-finite pattern differs"
    assert np.array_equal(got[~finite], ref[~finite]), "infinities differ"
    # 1e-30: results below it are at the edge of the fp32 range (softmax weights of
    # logits some 70 below the row maximum), where device arithmetic flushes to zero
    return float((np.abs(got[finite] - ref[finite]) / (mag[finite] + 1e-30)).max(initial=0.0))


_ERR_LOG = os.environ.get("GA_ERR_LOG")


def assert_close(got, ref, tol, what="", mag=None):
    """Norm criterion: max |got - ref| <= tol * max |ref|.  With ``mag`` also the
    element-wise one: |got_i - ref_i| <= tol * mag_i (see elementwise_err)."""
    err = rel_err(got, ref)
    err_el = elementwise_err(got, ref, mag) if mag is not None else None
    if _ERR_LOG:
        with open(_ERR_LOG, "a") as f:
            f.write(f"{what}\t{err:.3e}\t{'' if err_el is None else format(err_el, '.3e')}\t{tol:.1e}\n")
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol:.1e}"
    if err_el is not None:
        assert err_el <= tol, f"{what}: element-wise relative error {err_el:.3e} > {tol:.1e}"


def random_graph(rng, n, e):
    return (rng.integers(0, n, e, dtype=np.int64),
            rng.integers(0, n, e, dtype=np.int64))


def skewed_graph(rng, n, e, hub_deg):
    """Uniform edges plus one destination with ``hub_deg`` extra in-edges and a
    block of nodes without any in-edge; edge ids shuffled."""
    src, dst = random_graph(rng, n, e)
    dst = dst % (n // 2)                       # upper half: no in-edges
    hub = n // 3
    src = np.concatenate([src, rng.integers(0, n, hub_deg, dtype=np.int64)])
    dst = np.concatenate([dst, np.full(hub_deg, hub, np.int64)])
    perm = rng.permutation(src.shape[0])
    return src[perm], dst[perm]


def to_bf16_f32(a):
    """Round an fp32 numpy array to bf16 (nearest even) and return it as fp32."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)) \
        .to(torch.bfloat16).to(torch.float32).numpy()
