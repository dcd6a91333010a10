"""Fused sample loss (smx_sample_loss) through the C ABI against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.util import REL_F32, assert_close

pytestmark = pytest.mark.gpu


def _case(b, k, seed, spread=4.0):
    rng = np.random.default_rng(seed)
    f32 = lambda x: x.astype(np.float32).astype(np.float64)
    pos, neg = f32(rng.standard_normal(b) * spread), f32(rng.standard_normal((b, k)) * spread)
    mask = (rng.random((b, k)) > 0.25).astype(np.float64)
    w = f32(rng.random(b) + 0.1)
    return pos, neg, mask, w


@pytest.mark.parametrize("shape", [(1, 1), (7, 33), (64, 256), (300, 1000), (5, 4097)])
@pytest.mark.parametrize("temperature", [0.0, 1.0])
@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("masked", [False, True])
def test_sample_loss_matches_oracle(shape, temperature, weighted, masked):
    from smore_amd.training import sample_loss
    b, k = shape
    pos, neg, mask, w = _case(b, k, b * 1000 + k)
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    tp, tn = dev(pos).reshape(b, 1).requires_grad_(), dev(neg).requires_grad_()
    loss, pl, nl = sample_loss(tp, tn, dev(mask) if masked else None, dev(w) if weighted else None, temperature,
                               world_size=2)
    loss.backward()
    want = orc.sample_loss(pos, neg, mask if masked else None, w if weighted else None, temperature, 0.25)
    assert abs(pl.item() - want[0]) <= REL_F32 * abs(want[0]) and abs(nl.item() - want[1]) <= REL_F32 * abs(want[1])
    assert abs(loss.item() - 0.25 * (want[0] + want[1])) <= REL_F32 * abs(0.25 * (want[0] + want[1]))
    assert tp.grad.shape == (b, 1)
    assert_close(tp.grad.cpu().numpy().reshape(-1), want[2], REL_F32, "gradient of the positive logits")
    assert_close(tn.grad.cpu().numpy(), want[3], REL_F32, "gradient of the negative logits")


def test_saturated_logits_stay_finite():
    from smore_amd.training import sample_loss
    b, k = 4, 8
    neg = np.full((b, k), 90.0)
    neg[:, ::2] = -90.0
    pos = np.array([95.0, -95.0, 0.0, 30.0])
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    tp, tn = dev(pos).requires_grad_(), dev(neg).requires_grad_()
    loss, pl, nl = sample_loss(tp, tn, None, None, 1.0)
    loss.backward()
    want = orc.sample_loss(pos, neg, None, None, 1.0, 0.5)
    assert np.isfinite(loss.item()) and bool(torch.isfinite(tn.grad).all()) and bool(torch.isfinite(tp.grad).all())
    assert abs(pl.item() - want[0]) <= REL_F32 * abs(want[0]) and abs(nl.item() - want[1]) <= REL_F32 * abs(want[1])
    assert_close(tn.grad.cpu().numpy(), want[3], REL_F32, "gneg")


def test_loss_gradient_feeds_the_scoring_backward():
    """The gradient the loss pass writes is the upstream gradient of the fused scorer: one step of
    forward -> sample loss -> backward equals the oracle's chain."""
    from smore_amd import fused
    from smore_amd.training import sample_loss
    rng = np.random.default_rng(5)
    n, b, k, d = 500, 12, 40, 64
    f32 = lambda x: x.astype(np.float32).astype(np.float64)
    table, c = f32(rng.uniform(-0.07, 0.07, (n, d))), f32(rng.uniform(-0.07, 0.07, (b, d)))
    o = f32(np.abs(rng.uniform(-0.07, 0.07, (b, d))))
    idx = rng.integers(0, n, (b, k))
    pos = f32(rng.standard_normal(b))
    dev = lambda a: torch.tensor(a, dtype=torch.float32, device="cuda")
    t_table, t_c, t_o, t_idx = dev(table), dev(c), dev(o), torch.tensor(idx, device="cuda")
    params = fused.score_params(0.5, 0.02)   # small margin: logits near 0, gradients not saturated
    score = fused.score_forward("box", t_table, t_idx, t_c, t_o, params)
    tn = score.clone().requires_grad_()
    loss, _, _ = sample_loss(dev(pos), tn, None, None, 0.5)
    loss.backward()
    gq1, gq2 = fused.score_backward_query("box", t_table, t_idx, t_c, t_o, score, tn.grad.contiguous(), params)
    o_score = orc.score_forward("box", table[idx], c[:, None], o[:, None], 0.5, 0.02)
    _, _, _, o_gneg = orc.sample_loss(pos, o_score, None, None, 0.5, 0.5)
    _, o1, o2 = orc.score_backward("box", o_gneg, table[idx], c[:, None], o[:, None], 0.02)
    assert_close(gq1.cpu().numpy(), o1[:, 0], 2 * REL_F32, "center gradient through the loss")
    assert_close(gq2.cpu().numpy(), o2[:, 0], 2 * REL_F32, "offset gradient through the loss")


def test_argument_errors():
    from smore_amd import _lib
    from smore_amd.training import sample_loss
    neg = torch.zeros(3, 4, device="cuda")
    with pytest.raises(_lib.SmxError):
        sample_loss(torch.zeros(2, device="cuda"), neg)
    with pytest.raises(_lib.SmxError):
        sample_loss(torch.zeros(3, device="cuda"), neg, torch.zeros(3, 5, device="cuda"))
    with pytest.raises(_lib.SmxError):
        sample_loss(torch.zeros(3, device="cuda"), neg, adversarial_temperature=-1.0)
