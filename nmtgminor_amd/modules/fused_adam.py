"""FusedAdam on the multi-tensor HIP kernels, with the reference's class and constructor
(onmt/modules/optimized/fused_adam.py:4-191): Adam / AdamW whose elementwise update of ALL parameters of a group runs in
one launch per 48 tensors. Parameters may be fp16, bf16 or fp32 (the reference: fp16 and fp32); the moments have the
parameter's dtype, as in the reference; sparse gradients and AMSGrad are refused."""
import torch

from ..native import fused_optim


class MultiTensorApply(object):
    """Calls a fused_optim function with a fixed chunk size (fused_adam.py:4-31)."""
    available = True
    warned = False

    def __init__(self, chunk_size):
        self.chunk_size = chunk_size

    def check_avail(self):
        pass

    def __call__(self, op, noop_flag_buffer, tensor_lists, *args):
        return op(self.chunk_size, noop_flag_buffer, tensor_lists, *args)


multi_tensor_applier = MultiTensorApply(2048 * 32)


_SUPPORTED = (torch.float16, torch.bfloat16, torch.float32)


class FusedAdam(torch.optim.Optimizer):
    """Constructor arguments, defaults, param_group keys ('step' is kept per group) and state keys ('exp_avg', 'exp_avg_sq')
    are the reference's, so optimizer state_dicts interchange."""

    def __init__(self, params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, adam_w_mode=True, weight_decay=0.,
                 amsgrad=False, set_grad_none=True):
        if amsgrad:
            raise RuntimeError('FusedAdam does not support the AMSGrad variant.')
        super().__init__(params, dict(lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay))
        self.adam_w_mode = int(bool(adam_w_mode))
        self.set_grad_none = set_grad_none
        self._dummy_overflow_buf = None                       # the Adam pass raises no overflow flag
        self.multi_tensor_adam = fused_optim.multi_tensor_adam

    def zero_grad(self, set_to_none=True):
        if not set_to_none:
            return super().zero_grad(set_to_none=False)
        for group in self.param_groups:
            for param in group['params']:
                param.grad = None

    def _lists_by_dtype(self, group):
        """[grads, params, exp_avg, exp_avg_sq] per parameter dtype, for the parameters of the group that have a gradient;
        creates the moments of a parameter at its first step."""
        lists = {}
        for param in group['params']:
            grad = param.grad
            if grad is None:
                continue
            if grad.is_sparse:
                raise RuntimeError('FusedAdam does not support sparse gradients, please consider SparseAdam instead')
            if param.dtype not in _SUPPORTED:
                raise RuntimeError('FusedAdam only support fp16, bf16 and fp32.')
            if not param.is_contiguous():
                raise RuntimeError('FusedAdam needs contiguous parameters')
            state = self.state[param]
            if not state:
                for key in ('exp_avg', 'exp_avg_sq'):
                    state[key] = torch.zeros_like(param, memory_format=torch.contiguous_format)
            grad = (grad if grad.dtype == param.dtype else grad.to(param.dtype)).contiguous()
            for lst, t in zip(lists.setdefault(param.dtype, ([], [], [], [])), (grad, param, state['exp_avg'], state['exp_avg_sq'])):
                lst.append(t)
        return lists

    @torch.no_grad()
    def step(self, closure=None, grads=None, output_params=None, scale=None, grad_norms=None):
        if not all(arg is None for arg in (grads, output_params, scale, grad_norms)):
            raise RuntimeError('FusedAdam has been updated.  Simply initialize it identically to torch.optim.Adam, and call '
                               'step() with no arguments.')
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            group['step'] = group.get('step', 0) + 1
            beta1, beta2 = group['betas']
            for lists in self._lists_by_dtype(group).values():
                multi_tensor_applier(self.multi_tensor_adam, self._dummy_overflow_buf, list(lists), group['lr'], beta1, beta2,
                                     group['eps'], group['step'], self.adam_w_mode, int(bool(group['bias_correction'])),
                                     group['weight_decay'])
        return loss
