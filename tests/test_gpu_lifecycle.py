"""Library set-up and tear-down on the GPU: bpk_shutdown returns every byte bpk_init took."""
import pytest

pytestmark = pytest.mark.gpu


def test_init_shutdown_cycles_leave_device_memory_where_it_was():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from backpack_amd import capi
    L = capi.lib()
    capi.check(L.bpk_init(0))
    capi.check(L.bpk_shutdown())
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        capi.check(L.bpk_init(0))
        assert torch.cuda.mem_get_info()[0] < free0 - (128 << 20)     # the scratch areas exist
        capi.check(L.bpk_shutdown())
    assert torch.cuda.mem_get_info()[0] == free0, "bpk_init / bpk_shutdown leaks device memory"
    capi.check(L.bpk_init(0))       # the tests after this one find the library as they expect it
    x = torch.randn(4, 5000, device="cuda")
    idx = torch.empty(4, dtype=torch.int32, device="cuda")
    capi.check(L.bpk_argmax_rows(x.data_ptr(), 4, 5000, 5000, idx.data_ptr(), None, None))
    torch.cuda.synchronize()
    assert torch.equal(idx.long(), x.argmax(dim=1))
