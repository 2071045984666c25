"""bpk_argmax_rows_static, the entry point that allocates nothing: through the C ABI against
bpk_argmax_rows (the same kernel on allocated scratch) on the same logits — index work, exact — on two
calls in a row, the second smaller than the first, so that whatever the first call left in the shared
array would show."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from backpack_amd import capi
    capi.check(capi.lib().bpk_init(0))
    return capi.lib()


def _both(lib, lg):
    """(index, value) of bpk_argmax_rows and of bpk_argmax_rows_static on the same device logits."""
    import torch
    from backpack_amd import capi
    M, N = lg.shape
    d = torch.from_numpy(lg).cuda()
    s = torch.cuda.current_stream().cuda_stream
    outs = []
    for fn in (lib.bpk_argmax_rows, lib.bpk_argmax_rows_static):
        idx = torch.full((M,), -7, dtype=torch.int32, device="cuda")
        val = torch.full((M,), -7.0, dtype=torch.float32, device="cuda")
        capi.check(fn(d.data_ptr(), M, N, N, idx.data_ptr(), val.data_ptr(), s))
        outs.append((idx.cpu().numpy(), val.cpu().numpy()))
    return outs


def test_static_scratch_matches_allocated_scratch_twice_in_a_row(lib, kqo):
    rng = np.random.default_rng(0)
    # first call: 200 rows x 64 parts fill most of the array; second: fewer rows, fewer parts per row
    for M, N in ((200, 262144), (3, 9000), (256, 128256), (1, 1)):
        print("argmax static", M, N, flush=True)
        lg = rng.standard_normal((M, N)).astype(np.float32)
        if N > 100:
            lg[0, [5, N - 1]] = 11.0        # a tie across parts: the lowest index wins
        (i0, v0), (i1, v1) = _both(lib, lg)
        assert np.array_equal(i0, i1)
        assert np.array_equal(v0.view(np.uint32), v1.view(np.uint32))
        assert np.array_equal(i1, kqo.argmax_rows(lg))
        assert np.array_equal(v1, lg.max(axis=1))


def test_static_scratch_limit_and_mapped_memory_unchanged(lib):
    """More rows than the array holds are refused with a message; and a call changes neither the device
    memory in use nor what torch has reserved (nothing is allocated or freed)."""
    import torch
    from backpack_amd import capi
    lg = torch.randn(257, 1000, device="cuda")
    idx = torch.empty(257, dtype=torch.int32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    rc = lib.bpk_argmax_rows_static(lg.data_ptr(), 257, 1000, 1000, idx.data_ptr(), None, s)
    assert rc == -2 and b"256" in lib.bpk_last_error()
    capi.check(lib.bpk_argmax_rows_static(lg.data_ptr(), 256, 1000, 1000, idx.data_ptr(), None, s))
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for _ in range(10):
        capi.check(lib.bpk_argmax_rows_static(lg.data_ptr(), 256, 1000, 1000, idx.data_ptr(), None, s))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_reserved() == reserved0
    assert torch.equal(idx[:256].long(), lg[:256].argmax(dim=1))
