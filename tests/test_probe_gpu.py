"""The bandwidth probes move what they say they move (bench.py times them; here their effects are checked)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(kind, a, b, row_bytes=800, n_reads=1000):
    from smore_amd import _lib
    sink = torch.zeros(1, device="cuda")
    _lib.probe_bandwidth(kind, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
                         ctypes.c_void_p(a.data_ptr()), None if b is None else ctypes.c_void_p(b.data_ptr()),
                         a.numel() * a.element_size(), row_bytes, n_reads, ctypes.c_void_p(sink.data_ptr()))
    torch.cuda.synchronize()


@pytest.mark.parametrize("n", [1024, 1 << 20, (1 << 20) + 4 * 37])   # whole and ragged multiples of the unroll
def test_copy_update_fill_touch_every_element_once(n):
    a = torch.arange(n, dtype=torch.float32, device="cuda")
    b = torch.full((n,), -1.0, device="cuda")
    _run(2, a, b)
    assert torch.equal(b, a)
    _run(3, a, None)
    assert torch.equal(a, b * 2)
    _run(4, a, None)
    assert torch.equal(a.view(-1, 4), torch.tensor([1.0, 2.0, 3.0, 4.0], device="cuda").expand(n // 4, 4))


def test_read_and_row_probes_leave_memory_alone_and_check_arguments():
    from smore_amd import _lib
    a = torch.arange(1 << 18, dtype=torch.float32, device="cuda")
    keep = a.clone()
    for kind in (0, 1, 5, 6):
        _run(kind, a, None)
    _run(5, a, None, row_bytes=16, n_reads=8)
    _run(6, a, None, row_bytes=1024, n_reads=64)
    assert torch.equal(a, keep)
    with pytest.raises(_lib.SmxError):
        _run(5, a, None, row_bytes=40)          # not a multiple of 16
    with pytest.raises(_lib.SmxError):
        _run(2, a, None)                        # copy without destination
    with pytest.raises(_lib.SmxError):
        _run(9, a, None)
