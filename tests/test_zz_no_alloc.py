"""The entry point that allocates nothing (rsfk_symmetrize_count_noalloc) against the count-only call of
rsfk_symmetrize_device: identical row offsets and entry counts, on two calls in a row, the second with a smaller
input (the fixed working memory keeps the first call's contents), and refusal of inputs beyond its limits."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _graph(rng, N, K, torch):
    idx = rng.integers(0, N, size=(N, K)).astype(np.int32)
    idx[:, 0] = np.arange(N)
    idx[rng.random((N, K)) < 0.05] = -1                      # some empty slots
    # a row must not hold a point twice: blank the repeats
    srt = np.sort(idx, axis=1)
    order = np.argsort(idx, axis=1, kind="stable")
    dup = np.zeros_like(idx, dtype=bool)
    np.put_along_axis(dup, order[:, 1:], srt[:, 1:] == srt[:, :-1], axis=1)
    idx[dup] = -1
    return torch.from_numpy(idx).cuda()


def test_no_alloc_entry_point_matches_the_allocating_one(gpu):
    import torch
    rng = np.random.default_rng(11)
    for N, K, drop_self in [(200000, 32, True), (50000, 20, False), (777, 90, True)]:
        print("no-alloc symmetrize", N, K, drop_self, flush=True)
        d_idx = _graph(rng, N, K, torch)
        want = torch.empty(N + 1, dtype=torch.int32, device="cuda")
        got = torch.full((N + 1,), -7, dtype=torch.int32, device="cuda")
        nnz_want = gpu.symmetrize_device(d_idx.data_ptr(), 0, N, K, drop_self, want.data_ptr(), 0, 0, 0)
        nnz_got = gpu.symmetrize_count_noalloc(d_idx.data_ptr(), N, K, drop_self, got.data_ptr())
        torch.cuda.synchronize()
        assert nnz_got == nnz_want and nnz_got > 0
        assert torch.equal(got, want)
    with pytest.raises(gpu.RsfkError):
        gpu.symmetrize_count_noalloc(d_idx.data_ptr(), (1 << 20) + 1, 1, True, got.data_ptr())
    with pytest.raises(gpu.RsfkError):
        gpu.symmetrize_count_noalloc(d_idx.data_ptr(), 1 << 20, 64, True, got.data_ptr())
