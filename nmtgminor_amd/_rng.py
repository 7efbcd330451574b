"""Philox (seed, offset) pairs for kernels that draw their own dropout masks.

The pair comes from PyTorch's per-device default generator, whose offset is then advanced, the
way ATen ops reserve Philox counter space (the reference does the same under the generator's
mutex, onmt/modules/extensions/dropout_add/dropout.h:212-219)."""
import torch


def philox_seed_offset(device, n_elements):
    """Reserve counter space for n_elements draws; returns (seed, offset) as Python ints."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    gen = torch.cuda.default_generators[idx]
    seed = gen.initial_seed()
    offset = gen.get_offset()
    inc = ((int(n_elements) + 3) // 4) * 4
    gen.set_offset(offset + inc)
    return seed & 0xFFFFFFFFFFFFFFFF, offset


def philox4x32_10(counter, key):
    """Philox4x32-10 block function on Python ints: counter 4 words, key 2 words -> 4 words."""
    M0, M1, W0, W1, MASK = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85, 0xFFFFFFFF
    c = [w & MASK for w in counter]
    k0, k1 = key[0] & MASK, key[1] & MASK
    for _ in range(10):
        p0, p1 = M0 * c[0], M1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k0) & MASK, p1 & MASK, ((p0 >> 32) ^ c[3] ^ k1) & MASK, p0 & MASK]
        k0, k1 = (k0 + W0) & MASK, (k1 + W1) & MASK
    return c


def philox_keep_mask_reference(seed, offset, first, count, keep_p):
    """Pure-Python restatement of the device generator (tests only): keep flags of elements
    first .. first+count-1. Element e uses word e % 4 of the block whose counter is
    (offset_lo, offset_hi, (e/4)_lo, (e/4)_hi) under key (seed_lo, seed_hi)."""
    out = []
    cache = {}
    for e in range(first, first + count):
        b = e // 4
        if b not in cache:
            cache[b] = philox4x32_10([offset, offset >> 32, b, b >> 32], [seed, seed >> 32])
        u = (cache[b][e % 4] >> 8) * (1.0 / 16777216.0)
        out.append(1 if u < keep_p else 0)
    return out
