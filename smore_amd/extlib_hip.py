"""The `extlib_cuda` distance-operator function set on HIP.

Same names, argument order and in-place semantics as the pybind module of
smore/common/torchext/extlib_cuda.cpp:322-341 (declared :198-304): every
function writes into caller-allocated tensors and returns None.  Shapes are
derived exactly as dist_forward / dist_backward do (:172-196, :230-262):
be, ne from the entity tensor, bc, nc, dim from the first query tensor, the
output extents from dst / grad_out.  fp32 and fp64 are dispatched on the
entity dtype.  An unknown dist_type raises instead of printing and returning.
"""
import torch

from . import _lib


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _check(*tensors):
    dev = tensors[0].device
    if dev.type != "cuda":
        raise _lib.SmxError("smore_amd operators need device tensors (no CPU fallback)")
    for t in tensors:
        if t is None:
            continue
        if t.device != dev:
            raise _lib.SmxError("tensors on different devices")
        if not t.is_contiguous():
            raise _lib.SmxError("tensor is not contiguous")
        if t.dtype != tensors[0].dtype:
            raise _lib.SmxError("mixed dtypes")


def _suffix(t):
    if t.dtype == torch.float32:
        return "f32"
    if t.dtype == torch.float64:
        return "f64"
    raise _lib.SmxError(f"unsupported dtype {t.dtype}")


def _kind(name):
    k = _lib.load().smx_kind_from_name(name.encode())
    if k < 0:
        raise _lib.SmxError(f"unknown dist {name}")
    return k


def dist_forward(dname, entity_embed, first_embed, second_embed, dst, has_second):
    second = second_embed if has_second else None
    _check(entity_embed, first_embed, second, dst)
    be, ne = entity_embed.shape[0], entity_embed.shape[1]
    bc, nc, dim = first_embed.shape[0], first_embed.shape[1], first_embed.shape[2]
    bsize, num = dst.shape
    with torch.cuda.device(entity_embed.device):
        _lib.call(f"smx_dist_forward_{_suffix(entity_embed)}", _kind(dname), _stream(entity_embed),
                  _ptr(entity_embed), _ptr(first_embed), _ptr(second), _ptr(dst),
                  bsize, num, be, ne, bc, nc, dim)


def dist_backward(dname, grad_out, entity_embed, first_embed, second_embed, grad_entity, grad_first,
                  grad_second, has_second):
    second = second_embed if has_second else None
    gsecond = grad_second if has_second else None
    _check(grad_out, entity_embed, first_embed, second, grad_entity, grad_first, gsecond)
    be, ne = entity_embed.shape[0], entity_embed.shape[1]
    bc, nc, dim = first_embed.shape[0], first_embed.shape[1], first_embed.shape[2]
    bsize, num = grad_out.shape
    with torch.cuda.device(grad_out.device):
        _lib.call(f"smx_dist_backward_{_suffix(grad_out)}", _kind(dname), _stream(grad_out),
                  _ptr(grad_out), _ptr(entity_embed), _ptr(first_embed), _ptr(second),
                  _ptr(grad_entity), _ptr(grad_first), _ptr(gsecond),
                  bsize, num, be, ne, bc, nc, dim)


def box_dist_forward(entity_embed, center_embed, offset_embed, dst, dist_type):
    dist_forward("box_" + dist_type, entity_embed, center_embed, offset_embed, dst, True)


def box_dist_backward(grad_out, entity_embed, center_embed, offset_embed, grad_entity, grad_center,
                      grad_offset, dist_type):
    dist_backward("box_" + dist_type, grad_out, entity_embed, center_embed, offset_embed,
                  grad_entity, grad_center, grad_offset, True)


def rotate_dist_forward(entity_embed, re_embed, im_embed, dst):
    dist_forward("rotate", entity_embed, re_embed, im_embed, dst, True)


def rotate_dist_backward(grad_out, entity_embed, re_embed, im_embed, grad_entity, grad_re, grad_im):
    dist_backward("rotate", grad_out, entity_embed, re_embed, im_embed, grad_entity, grad_re, grad_im, True)


def l1_dist_forward(entity_embed, center_embed, dst):
    dist_forward("l1", entity_embed, center_embed, None, dst, False)


def l1_dist_backward(grad_out, entity_embed, center_embed, grad_entity, grad_center):
    dist_backward("l1", grad_out, entity_embed, center_embed, None, grad_entity, grad_center, None, False)


def l2_dist_forward(entity_embed, center_embed, dst):
    dist_forward("l2", entity_embed, center_embed, None, dst, False)


def l2_dist_backward(grad_out, entity_embed, center_embed, grad_entity, grad_center):
    dist_backward("l2", grad_out, entity_embed, center_embed, None, grad_entity, grad_center, None, False)


def complex_dist_forward(entity_embed, re_embed, im_embed, dst):
    dist_forward("complex", entity_embed, re_embed, im_embed, dst, True)


def complex_dist_backward(grad_out, entity_embed, re_embed, im_embed, grad_entity, grad_re, grad_im):
    dist_backward("complex", grad_out, entity_embed, re_embed, im_embed, grad_entity, grad_re, grad_im, True)


def beta_dist_forward(entity_embed, re_embed, im_embed, dst, dist_type):
    dist_forward("beta_" + dist_type, entity_embed, re_embed, im_embed, dst, True)


def beta_dist_backward(grad_out, entity_embed, re_embed, im_embed, grad_entity, grad_re, grad_im, dist_type):
    dist_backward("beta_" + dist_type, grad_out, entity_embed, re_embed, im_embed, grad_entity, grad_re,
                  grad_im, True)


def distmult_dist_forward(entity_embed, center_embed, dst):
    dist_forward("distmult", entity_embed, center_embed, None, dst, False)


def distmult_dist_backward(grad_out, entity_embed, center_embed, grad_entity, grad_center):
    dist_backward("distmult", grad_out, entity_embed, center_embed, None, grad_entity, grad_center, None, False)
