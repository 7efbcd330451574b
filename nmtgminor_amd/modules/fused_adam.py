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


class FusedAdam(torch.optim.Optimizer):
    def __init__(self, params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, adam_w_mode=True, weight_decay=0.,
                 amsgrad=False, set_grad_none=True):
        if amsgrad:
            raise RuntimeError('FusedAdam does not support the AMSGrad variant.')
        defaults = dict(lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay)
        super(FusedAdam, self).__init__(params, defaults)
        self.adam_w_mode = 1 if adam_w_mode else 0
        self.set_grad_none = set_grad_none
        self._dummy_overflow_buf = None
        self.multi_tensor_adam = fused_optim.multi_tensor_adam

    def zero_grad(self, set_to_none=True):
        if set_to_none:
            for group in self.param_groups:
                for p in group['params']:
                    p.grad = None
        else:
            super(FusedAdam, self).zero_grad()

    @torch.no_grad()
    def step(self, closure=None, grads=None, output_params=None, scale=None, grad_norms=None):
        if any(p is not None for p in [grads, output_params, scale, grad_norms]):
            raise RuntimeError('FusedAdam has been updated.  Simply initialize it identically to torch.optim.Adam, and call '
                               'step() with no arguments.')
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            bias_correction = 1 if group['bias_correction'] else 0
            beta1, beta2 = group['betas']
            group['step'] = group.get('step', 0) + 1
            by_dtype = {}
            for p in group['params']:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError('FusedAdam does not support sparse gradients, please consider SparseAdam instead')
                if p.dtype not in (torch.float16, torch.bfloat16, torch.float32):
                    raise RuntimeError('FusedAdam only support fp16, bf16 and fp32.')
                state = self.state[p]
                if len(state) == 0:
                    state['exp_avg'] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                    state['exp_avg_sq'] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                if not p.is_contiguous():
                    raise RuntimeError('FusedAdam needs contiguous parameters')
                lists = by_dtype.setdefault(p.dtype, ([], [], [], []))
                g = p.grad if p.grad.dtype == p.dtype else p.grad.to(p.dtype)
                for lst, t in zip(lists, (g.contiguous(), p, state['exp_avg'], state['exp_avg_sq'])):
                    lst.append(t)
            for lists in by_dtype.values():
                multi_tensor_applier(self.multi_tensor_adam, self._dummy_overflow_buf, list(lists), group['lr'], beta1, beta2,
                                     group['eps'], group['step'], self.adam_w_mode, bias_correction, group['weight_decay'])
        return loss
