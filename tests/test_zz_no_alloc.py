"""pcm_pairwise_mi_static -- the entry point that allocates nothing -- against pcm_pairwise_mi:
the same kernels on a fixed array of the library instead of freshly allocated buffers, so the
results must be bit-identical.  Two calls in a row, the second smaller (the array keeps the first
call's bytes), then the size limits."""
import numpy as np
import pytest

from test_structure import _data


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355
    return torch, pcmi355


def _both(torch, P, x, C, pc):
    from pcmi355._lib import lib, check
    d = torch.from_numpy(x).cuda()
    n, v = x.shape
    stream = torch.cuda.current_stream().cuda_stream
    want = torch.full((v, v), -7.0, dtype=torch.float32, device="cuda")
    got = torch.full((v, v), -9.0, dtype=torch.float32, device="cuda")
    check(lib.pcm_pairwise_mi(d.data_ptr(), d.stride(0), d.stride(1), n, v, C, pc, want.data_ptr(), stream))
    check(lib.pcm_pairwise_mi_static(d.data_ptr(), d.stride(0), d.stride(1), n, v, C, pc, got.data_ptr(), stream))
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


@pytest.mark.gpu
def test_static_entry_point_matches_the_allocating_one_twice(gpu):
    torch, P = gpu
    import structure_oracle as S
    print("pcm_pairwise_mi_static: first call 3000 x 40 x 256", flush=True)
    x1 = _data(3000, 40, 256, 5)
    got1, want1 = _both(torch, P, x1, 256, 0.1)
    assert np.array_equal(got1, want1)                      # bit-exact: same kernels, same order of sums
    print("pcm_pairwise_mi_static: second, smaller call 700 x 9 x 16", flush=True)
    x2 = _data(700, 9, 16, 6)
    got2, want2 = _both(torch, P, x2, 16, 0.0)
    assert np.array_equal(got2, want2)
    ref = S.pairwise_mi(x2, 16, 0.0)
    assert np.abs(got2 - ref).max() < 1e-4 * np.abs(ref).max()
    # and a larger one again after the small one
    got3, want3 = _both(torch, P, x1[:2999], 256, 0.5)
    assert np.array_equal(got3, want3)


@pytest.mark.gpu
def test_static_entry_point_allocates_nothing_and_takes_any_stream(gpu):
    """After one warm-up call (the first call on a device resolves the array's address), further calls leave the
    device's free memory as it was -- hipMemGetInfo, with torch's caching allocator idle --, and a call queued on a
    stream of the caller's gives the same bits as one on the default stream."""
    torch, P = gpu
    from pcmi355._lib import lib, check
    x = _data(2000, 24, 64, 11)
    d = torch.from_numpy(x).cuda()
    n, v = x.shape
    out0 = torch.zeros((v, v), dtype=torch.float32, device="cuda")
    out1 = torch.zeros((v, v), dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    check(lib.pcm_pairwise_mi_static(d.data_ptr(), d.stride(0), d.stride(1), n, v, 64, 0.1, out0.data_ptr(), None))   # warm-up
    torch.cuda.synchronize()
    # (the runtime sets a new stream up at its first launch; that is the stream's cost, not the entry point's)
    check(lib.pcm_pairwise_mi_static(d.data_ptr(), d.stride(0), d.stride(1), n, v, 64, 0.1, out1.data_ptr(), side.cuda_stream))
    side.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        check(lib.pcm_pairwise_mi_static(d.data_ptr(), d.stride(0), d.stride(1), n, v, 64, 0.1, out0.data_ptr(), None))
    torch.cuda.synchronize()
    check(lib.pcm_pairwise_mi_static(d.data_ptr(), d.stride(0), d.stride(1), n, v, 64, 0.1, out1.data_ptr(), side.cuda_stream))
    side.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(out0, out1)


@pytest.mark.gpu
def test_static_entry_point_rejects_what_its_array_cannot_hold(gpu):
    torch, P = gpu
    from pcmi355._lib import lib
    out = torch.zeros((2, 2), dtype=torch.float32, device="cuda")
    big = torch.zeros((65536, 2), dtype=torch.uint8, device="cuda")
    assert lib.pcm_pairwise_mi_static(big.data_ptr(), 2, 1, 65536, 2, 4, 0.1, out.data_ptr(), None) == -3
    assert b"65535" in lib.pcm_last_error()
    wide = torch.zeros((8, 4097), dtype=torch.uint8, device="cuda")
    assert lib.pcm_pairwise_mi_static(wide.data_ptr(), 4097, 1, 8, 4097, 4, 0.1, out.data_ptr(), None) == -3
    # 4096 variables x 4160 staged examples = 17 039 360 bytes > 16 MiB
    tall = torch.zeros((4100, 4096), dtype=torch.uint8, device="cuda")
    assert lib.pcm_pairwise_mi_static(tall.data_ptr(), 4096, 1, 4100, 4096, 4, 0.1, out.data_ptr(), None) == -3
    assert b"static buffer" in lib.pcm_last_error()
    torch.cuda.synchronize()
