"""Gradient clipping by the global L2 norm on the multi-tensor kernels, with the reference's function
(onmt/modules/optimized/fused_clip_norm.py:20-138): one norm pass over all gradients of a dtype and one scaling pass,
instead of one small kernel per parameter. Same result as torch.nn.utils.clip_grad_norm_ for the 2-norm. Other norms and
gradients that are not on the GPU have no HIP path and raise (the reference falls back to a per-tensor loop there)."""
import torch

from ..native import fused_optim
from .fused_adam import multi_tensor_applier


def fused_clip_grad_norm(parameters, max_norm, norm_type=2.0, error_if_nonfinite=False):
    """Clips the gradients of `parameters` in place so that their joint L2 norm is at most max_norm (no scaling if
    max_norm <= 0). -> the joint norm before clipping (fp32 tensor on the gradients' device)."""
    if isinstance(parameters, torch.Tensor):
        parameters = [parameters]
    parameters = [p for p in parameters if p.grad is not None]
    max_norm, norm_type = float(max_norm), float(norm_type)
    if len(parameters) == 0:
        return torch.tensor(0.)
    if norm_type != 2.0:
        raise NotImplementedError("fused_clip_grad_norm: only the 2-norm has a HIP kernel")
    device = parameters[0].grad.device
    by_dtype = {}
    for p in parameters:
        grad = p.grad.detach()
        if grad.device != device or grad.dtype not in (torch.float32, torch.float16, torch.bfloat16) or not grad.is_contiguous():
            raise RuntimeError("fused_clip_grad_norm: gradients must be contiguous fp32 / fp16 / bf16 tensors on one device")
        by_dtype.setdefault(grad.dtype, []).append(grad)
    dummy_overflow_buf = torch.zeros([1], dtype=torch.int32, device=device)
    norms = [multi_tensor_applier(fused_optim.multi_tensor_l2norm, dummy_overflow_buf, [grads], False)[0]
             for grads in by_dtype.values()]
    if len(norms) == 1:
        total_norm = norms[0][0]
    else:
        # the joint norm of at most three partial norms, through the same kernel
        total_norm = multi_tensor_applier(fused_optim.multi_tensor_l2norm, dummy_overflow_buf, [[torch.cat(norms)]], False)[0][0]
    if error_if_nonfinite and not bool(torch.isfinite(total_norm)):
        raise RuntimeError(f'The total norm of order {norm_type} for gradients from `parameters` is non-finite, so it cannot be '
                           'clipped. To disable this error and scale the gradients by the non-finite norm anyway, set '
                           '`error_if_nonfinite=False`')
    if max_norm > 0:
        # the clipping factor is computed in fp32 like the reference's tensor expression; reading it back is the one
        # host synchronisation of the function (the reference's float conversion of the same tensor)
        clip_coef = float(torch.clamp(max_norm / (total_norm + 1e-6), max=1.0))
        for grads in by_dtype.values():
            multi_tensor_applier(fused_optim.multi_tensor_scale, dummy_overflow_buf, [grads, grads], clip_coef)
    return total_norm
