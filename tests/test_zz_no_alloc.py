"""The entry point that allocates nothing (rsfk_symmetrize_count_noalloc) against the count-only call of
rsfk_symmetrize_device: identical row offsets and entry counts, on two calls in a row, the second with a smaller
input (the fixed working memory keeps the first call's contents), the form that leaves the count on the device, the
amount of free device memory before and after, and refusal of inputs beyond its limits."""
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
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        nnz_got = gpu.symmetrize_count_noalloc(d_idx.data_ptr(), N, K, drop_self, got.data_ptr())
        torch.cuda.synchronize()
        # the device's free memory did not move (the allocating call would take 7 MB and more for the first input;
        # the slack is for the runtime's own small pools)
        assert abs(torch.cuda.mem_get_info()[0] - free_before) <= (1 << 20)
        assert nnz_got == nnz_want and nnz_got > 0
        assert torch.equal(got, want)
        # the form that only enqueues kernels: no count comes back, it is the last row offset on the device
        got.fill_(-7)
        assert gpu.symmetrize_count_noalloc(d_idx.data_ptr(), N, K, drop_self, got.data_ptr(), fetch_count=False) is None
        torch.cuda.synchronize()
        assert abs(torch.cuda.mem_get_info()[0] - free_before) <= (1 << 20)
        assert torch.equal(got, want) and int(got[N]) == nnz_want
    with pytest.raises(gpu.RsfkError):
        gpu.symmetrize_count_noalloc(d_idx.data_ptr(), (1 << 20) + 1, 1, True, got.data_ptr())
    with pytest.raises(gpu.RsfkError):
        gpu.symmetrize_count_noalloc(d_idx.data_ptr(), 1 << 20, 64, True, got.data_ptr())
