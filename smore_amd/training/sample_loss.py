"""The sample loss of a training step (smore/training/train_process.py:194-213) as one fused pass.

`sample_loss` returns the two logged losses and the differentiable total; its backward hands autograd
the gradients the forward pass already computed, so the dozen element-wise kernels of the reference's
formulation (mask multiply, softmax, logsigmoid, weighted sums, and their autograd twins) become one
launch over the [B,K] logits."""
import ctypes

import torch

from .. import _lib
from ..fused import _ptr, _stream, _workspace


class _SampleLossFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, pos, neg, mask, weight, temperature, scale):
        b, k = neg.shape
        out = torch.empty(2, dtype=torch.float32, device=neg.device)
        gpos = torch.empty(b, dtype=torch.float32, device=neg.device)
        gneg = torch.empty((b, k), dtype=torch.float32, device=neg.device)
        with torch.cuda.device(neg.device):
            ws = _workspace(_lib.load().smx_sample_loss_workspace_bytes(b), neg.device)
            _lib.call("smx_sample_loss", _stream(neg), _ptr(pos), _ptr(neg), _ptr(mask), _ptr(weight), b, k,
                      ctypes.c_double(temperature), ctypes.c_double(scale), _ptr(out), _ptr(gpos), _ptr(gneg),
                      _ptr(ws), ws.numel())
        ctx.save_for_backward(gpos, gneg)
        ctx.pos_shape = pos.shape
        ctx.mark_non_differentiable(out)
        return (out[0] + out[1]) * scale, out

    @staticmethod
    def backward(ctx, g_total, _g_out):
        gpos, gneg = ctx.saved_tensors
        return (gpos * g_total).reshape(ctx.pos_shape), gneg * g_total, None, None, None, None


def sample_loss(positive_logit, negative_logit, is_negative_mat=None, subsampling_weight=None,
                adversarial_temperature=0.0, world_size=1):
    """positive_logit [B] or [B,1], negative_logit [B,K] (fp32, device); is_negative_mat [B,K] or None;
    subsampling_weight [B] or None ('u' mode); adversarial_temperature 0 = --negative_adversarial_sampling off.
    Returns (loss, positive_sample_loss, negative_sample_loss): loss = (pos + neg) / 2 / world_size carries
    the gradient (add reg_loss * reg_coeff / 2 / world_size to it as the reference does); the other two are
    the detached values the reference logs."""
    def prep(t, name):
        if t is None:
            return None
        if t.dtype != torch.float32 or t.device != negative_logit.device:
            raise _lib.SmxError(f"{name} must be a float32 tensor on the logits' device")
        return t.contiguous()
    if negative_logit.dim() != 2 or negative_logit.device.type != "cuda":
        raise _lib.SmxError("negative_logit must be a [B,K] device tensor")
    b, k = negative_logit.shape
    pos = prep(positive_logit, "positive_logit")
    if pos.numel() != b:
        raise _lib.SmxError("positive_logit must hold one value per query")
    mask = prep(is_negative_mat, "is_negative_mat")
    if mask is not None and mask.shape != negative_logit.shape:
        raise _lib.SmxError("is_negative_mat must have the shape of negative_logit")
    weight = prep(subsampling_weight, "subsampling_weight")
    if weight is not None and weight.numel() != b:
        raise _lib.SmxError("subsampling_weight must hold one value per query")
    total, parts = _SampleLossFunc.apply(pos, prep(negative_logit, "negative_logit"), mask, weight,
                                         float(adversarial_temperature), 0.5 / float(world_size))
    return total, parts[0], parts[1]
