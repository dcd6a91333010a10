"""smx_sample_loss_static (scratch in a static device array, no allocation) through the C ABI against
smx_sample_loss: same bits, on two calls in a row, the second with a smaller input."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_QUERIES = 65536


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _both(b, k, seed, weighted, masked, temperature):
    from smore_amd import _lib
    lib = _lib.load()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    pos = torch.randn(b, device="cuda", generator=gen) * 3
    neg = torch.randn((b, k), device="cuda", generator=gen) * 3
    mask = (torch.rand((b, k), device="cuda", generator=gen) > 0.25).float() if masked else None
    weight = torch.rand(b, device="cuda", generator=gen) + 0.1 if weighted else None
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for static in (False, True):
        loss = torch.full((2,), float("nan"), device="cuda")
        gpos = torch.full((b,), float("nan"), device="cuda")
        gneg = torch.full((b, k), float("nan"), device="cuda")
        args = [stream, _ptr(pos), _ptr(neg), _ptr(mask), _ptr(weight), b, k, ctypes.c_double(temperature),
                ctypes.c_double(0.5), _ptr(loss), _ptr(gpos), _ptr(gneg)]
        if static:
            _lib.call("smx_sample_loss_static", *args)
        else:
            ws = torch.empty(lib.smx_sample_loss_workspace_bytes(b), dtype=torch.uint8, device="cuda")
            _lib.call("smx_sample_loss", *args, _ptr(ws), ws.numel())
        torch.cuda.synchronize()
        out.append((loss, gpos, gneg))
    for name, a, c in zip(("loss", "gpos", "gneg"), *out):
        assert bool(torch.isfinite(a).all()), name
        assert torch.equal(a, c), f"{name}: the static-scratch call differs from smx_sample_loss (B={b}, K={k})"


@pytest.mark.parametrize("weighted,masked,temperature", [(True, True, 1.0), (False, False, 0.0), (True, False, 0.5)])
def test_static_scratch_loss_matches_the_workspace_call(weighted, masked, temperature):
    print("case: smx_sample_loss_static B=700,K=300 then B=37,K=129", weighted, masked, temperature, flush=True)
    _both(700, 300, 11, weighted, masked, temperature)
    _both(37, 129, 12, weighted, masked, temperature)      # smaller: the array still holds the first call's values


def test_static_scratch_loss_rejects_batches_beyond_its_array():
    from smore_amd import _lib
    x = torch.zeros(4, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    with pytest.raises(_lib.SmxError, match="at most"):
        _lib.call("smx_sample_loss_static", stream, _ptr(x), _ptr(x), None, None, MAX_QUERIES + 1, 1,
                  ctypes.c_double(0.0), ctypes.c_double(0.5), _ptr(x), _ptr(x), _ptr(x))
