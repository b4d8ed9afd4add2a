"""k-means on the device against the CPU checker and against an fp64 brute force."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from gpu_helpers import dev, gaussian_mixture
from vsag_amd import capi

pytestmark = pytest.mark.gpu


def gpu_assign(x, cent):
    L = capi.load_library()
    n, d = x.shape
    k = cent.shape[0]
    xb, cb = dev(x), dev(cent)
    labels, mind, loss = capi.DeviceBuffer(n * 4), capi.DeviceBuffer(n * 4), capi.DeviceBuffer(8)
    wsb = L.vsag_amd_kmeans_assign_workspace_bytes(n, d, k)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_kmeans_assign(xb.ptr, n, d, cb.ptr, k, labels.ptr, mind.ptr, loss.ptr, ws.ptr, wsb, None))
    return labels.to_numpy(np.int32, (n,)), mind.to_numpy(np.float32, (n,)), float(loss.to_numpy(np.float64, (1,))[0])


def check_assignment(x, cent, labels, mind, rel=1e-5):
    """labels must be the exact argmin except where the runner-up is within rel of the winner."""
    x64, c64 = x.astype(np.float64), cent.astype(np.float64)
    d2 = (c64 ** 2).sum(1)[None, :] - 2.0 * x64 @ c64.T
    best = d2.argmin(1)
    scale = (x64 ** 2).sum(1) + np.abs(d2.min(1))
    chosen = d2[np.arange(len(x)), labels]
    wrong = labels != best
    gap = chosen - d2.min(1)
    assert np.all(gap[wrong] <= rel * scale[wrong]), "assignment differs outside the near-tie band: %d rows" % int(
        (gap > rel * scale).sum())
    assert np.allclose(mind, d2.min(1), rtol=1e-4, atol=1e-4 * scale.max())
    return int(wrong.sum())


@pytest.mark.parametrize("n,d,k", [(3000, 128, 100), (1000, 960, 257), (129, 7, 3), (5000, 33, 1000), (64, 16, 64),
                                   (3000, 100, 100), (2000, 104, 500), (1500, 12, 40)])
def test_assign_matches_bruteforce_and_oracle(lib, n, d, k):
    rng = np.random.default_rng(n + d + k)
    x, _ = gaussian_mixture(rng, n, d, max(2, k // 4), 0.2, uniform_means=False)
    cent = x[rng.choice(n, k, replace=False)].copy()
    labels, mind, loss = gpu_assign(x, cent)
    assert labels.min() >= 0 and labels.max() < k
    check_assignment(x, cent, labels, mind)
    olabels, omind, oloss = orc.kmeans_assign(x, cent)
    agree = (labels == olabels).mean()
    assert agree > 0.999, agree
    assert abs(loss - oloss) <= 1e-4 * abs(oloss) + 1e-6


def test_first_minimum_wins_ties(lib):
    # duplicated centroids: std::min_element keeps the first of equal minima
    rng = np.random.default_rng(3)
    x = rng.standard_normal((500, 32)).astype(np.float32)
    base = rng.standard_normal((40, 32)).astype(np.float32)
    cent = np.concatenate([base, base, base]).astype(np.float32)
    labels, _, _ = gpu_assign(x, cent)
    assert labels.max() < 40


@pytest.mark.parametrize("n,d,k", [(4000, 64, 50), (700, 960, 9)])
def test_update_matches_oracle(lib, n, d, k):
    L = lib.load_library()
    rng = np.random.default_rng(n + k)
    x = rng.standard_normal((n, d)).astype(np.float32)
    labels = rng.integers(0, k, n).astype(np.int32)
    labels[labels == 3] = 4  # cluster 3 is empty
    cent0 = rng.standard_normal((k, d)).astype(np.float32)
    xb, lb, cb = dev(x), dev(labels), dev(cent0)
    counts = capi.DeviceBuffer(k * 4)
    wsb = L.vsag_amd_kmeans_update_workspace_bytes(n, d, k)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_kmeans_update(xb.ptr, lb.ptr, n, d, k, cb.ptr, counts.ptr, ws.ptr, wsb, None))
    cent = cb.to_numpy(np.float32, (k, d))
    cnt = counts.to_numpy(np.int32, (k,))
    rcent, rcnt = orc.kmeans_update(x, labels, cent0)
    assert np.array_equal(cnt, rcnt) and cnt[3] == 0
    assert np.array_equal(cent[3], cent0[3])  # empty cluster untouched
    assert np.allclose(cent, rcent, rtol=1e-5, atol=1e-6)


def test_run_matches_oracle_and_reduces_loss(lib):
    L = lib.load_library()
    rng = np.random.default_rng(11)
    n, d, k, iters = 6000, 48, 64, 6
    x, _ = gaussian_mixture(rng, n, d, 64, 0.2, uniform_means=False)
    cent0 = x[rng.choice(n, k, replace=False)].copy()
    xb, cb = dev(x), dev(cent0)
    labels = capi.DeviceBuffer(n * 4)
    loss = C.c_double()
    wsb = L.vsag_amd_kmeans_run_workspace_bytes(n, d, k)
    ws = capi.DeviceBuffer(wsb)
    capi.check(L.vsag_amd_kmeans_run(xb.ptr, n, d, cb.ptr, k, iters, 7, labels.ptr, C.byref(loss), ws.ptr, wsb, None))
    cent = cb.to_numpy(np.float32, (k, d))
    rcent, rlabels, rloss = orc.kmeans_run(x, cent0, iters, 7)
    _, _, loss0 = orc.kmeans_assign(x, cent0)
    assert loss.value < loss0
    assert abs(loss.value - rloss) <= 1e-3 * abs(rloss)
    assert (labels.to_numpy(np.int32, (n,)) == rlabels).mean() > 0.99
    assert np.allclose(cent, rcent, rtol=1e-3, atol=1e-3)


def test_kmeans_argument_errors(lib):
    L = lib.load_library()
    x = dev(np.zeros((4, 4), np.float32))
    rc = L.vsag_amd_kmeans_run(x.ptr, 4, 4, x.ptr, 8, 1, 0, x.ptr, None, None, 0, None)
    assert rc == capi.INVALID_ARGUMENT and b"k cannot be larger than count" in L.vsag_amd_last_error()
    rc = L.vsag_amd_kmeans_assign(x.ptr, 4, 4, x.ptr, 0, x.ptr, None, None, None, 0, None)
    assert rc == capi.INVALID_ARGUMENT and b"k must be positive" in L.vsag_amd_last_error()


def gpu_init_pp(x, k, first, draws):
    L = capi.load_library()
    n, d = x.shape
    xb = dev(x)
    cent, picks = capi.DeviceBuffer(k * d * 4), capi.DeviceBuffer(k * 8)
    wsb = L.vsag_amd_kmeans_init_plus_plus_workspace_bytes(n)
    ws = capi.DeviceBuffer(wsb)
    draws = np.ascontiguousarray(draws, np.float64)
    capi.check(L.vsag_amd_kmeans_init_plus_plus(xb.ptr, n, d, k, first, draws.ctypes.data, cent.ptr, picks.ptr, ws.ptr,
                                                wsb, None))
    capi.synchronize()
    out = cent.to_numpy(np.float32, (k, d)), picks.to_numpy(np.uint64, (k,))
    for b in (xb, cent, picks, ws):
        b.free()
    return out


@pytest.mark.parametrize("n,d,k", [(5000, 128, 64), (777, 7, 100), (20000, 65, 33), (64, 960, 64), (130, 16, 130)])
def test_plus_plus_seeding_matches_oracle(lib, n, d, k):
    """k-means++ seeding (kmeans_cluster.cpp:383-435) with the same draws as the checker: the same rows, except where a
    threshold falls within the rounding of the (differently associated) double sums of a boundary."""
    rng = np.random.default_rng(n + d + k)
    x, _ = gaussian_mixture(rng, n, d, max(2, k // 4), 0.2, uniform_means=False)
    draws = rng.random(k - 1)
    first = int(rng.integers(n))
    cent, picks = gpu_init_pp(x, k, first, draws)
    rcent, rpicks = orc.kmeans_init_pp(x, k, first, draws)
    assert np.array_equal(picks, rpicks), np.nonzero(picks != rpicks)[0][:5]
    assert np.array_equal(cent, rcent)
    assert len(set(picks.tolist())) == k


def test_plus_plus_seeding_on_coincident_rows(lib):
    rng = np.random.default_rng(4)
    y = np.repeat(rng.standard_normal((3, 20)).astype(np.float32), 50, axis=0)
    draws = np.array([0.5, 0.99, 0.0, 0.5, 0.999])
    cent, picks = gpu_init_pp(y, 6, 0, draws)
    _, rpicks = orc.kmeans_init_pp(y, 6, 0, draws)
    assert np.array_equal(picks, rpicks) and list(picks[3:]) == [0, 75, 149]
    L = capi.load_library()
    assert L.vsag_amd_kmeans_init_plus_plus(1, 10, 4, 3, 10, draws.ctypes.data, 1, None, None, 0, None) == capi.INVALID_ARGUMENT
