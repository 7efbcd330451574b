"""Autocast handling shared by the op wrappers: under autocast, floating-point tensor arguments
are cast to the autocast dtype and the op itself runs with autocast disabled (what the reference
does around every fused op, e.g. onmt/modules/optimized/self_attention_func.py:507-520)."""
import torch


def cast_if_autocast_enabled(*args):
    if not torch.is_autocast_enabled():
        return args
    dtype = torch.get_autocast_dtype("cuda")
    return torch.amp.autocast_mode._cast(args, "cuda", dtype)


def no_autocast():
    return torch.amp.autocast("cuda", enabled=False)
