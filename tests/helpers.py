"""Shared helpers for the parity tests."""
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


def assert_close(got, ref, tol, what=""):
    err = rel_err(got, ref)
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol:.1e}"


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
