"""Output projection + label-smoothed cross-entropy: the logits are kept once, in the working dtype, when they fit a
stated budget of device memory, and never materialised otherwise.

The reference projects the decoder states to the vocabulary (Generator.forward,
onmt/modules/base_seq2seq.py:26-47) and hands the whole logits tensor to the loss
(CrossEntropyLossBase._compute_loss, onmt/modules/loss.py:60-109, which calls
SoftmaxCrossEntropyLoss.apply(logits, labels, smoothing, padding_idx, half_to_float)). At a vocabulary of 250 054 and
16 384 target positions that tensor and its gradient are 8.2 GB each. Here the same two kernels (the MFMA projection and
the cross-entropy) run over pieces of it. The forward walks the rows `chunk_rows` at a time (a row's log-sum-exp needs
the whole row) and keeps only the per-row losses and log-sum-exp. The backward is elementwise once the log-sum-exp is
known, so it walks the vocabulary in column slices over all rows: it recomputes a slice's logits, turns them into
their gradient and contracts that at once with the states (the slice's weight gradient: complete, written once) and
with the slice's weights (gradient of the states, [N, E], summed over the slices in fp32). Per-row results are those of
the unchunked pair of operators to rounding; arbitrary per-row upstream gradients (loss weights) are supported because
nothing of the backward is precomputed in the forward.

Kept logits (`keep_logits_bytes`, default 16 GiB): a training call whose [N, V] logits fit the budget (8.2 GB for the
case above; this GPU has 288 GB) projects once over all rows, keeps the logits for the backward and turns them into their
gradient in place there, which is then contracted once with the states (the weight gradient) and once with the weights
(the gradient of the states): three products of N x E x V per step instead of four, and one tensor of the logits' size
where the reference holds two (the logits saved by autograd and their gradient, xentropy_kernel.cu:636-645). A second
backward over the same graph finds the logits consumed and takes the recomputing path.

The chunk buffers have a row pitch of the vocabulary rounded up to 64 elements, so that the projection's stores and the
two contractions that read the logits gradient move 16 bytes per access whatever the vocabulary size (250 054 is not a
multiple of 4); the cross-entropy kernels read and write the first V elements of each pitched row in place.

Beyond the kernels (projection, cross-entropy, column sums for the bias gradient) this module only slices and sums the
per-slice gradients of the states (`add_` in fp32, [N, E]): a device-side PyTorch call on already computed pieces.
"""
import torch
import torch.nn as nn

from ..native import linear_gemm, xentropy_cuda

DEFAULT_CHUNK_ROWS = 4096
DEFAULT_KEEP_LOGITS_BYTES = 16 << 30


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _check_inputs(hidden, weight, bias, labels, chunk_rows):
    _check(hidden.dim() == 2 and weight.dim() == 2, "hidden must be [N, E] and weight [V, E]")
    _check(hidden.size(1) == weight.size(1), "hidden and weight disagree on the model dimension")
    _check(hidden.dtype in (torch.float16, torch.bfloat16) and weight.dtype == hidden.dtype,
           "fp16 or bf16 states and weights of one dtype required")
    _check(bias is None or (bias.dim() == 1 and bias.size(0) == weight.size(0) and bias.dtype == hidden.dtype),
           "bias must be [V] in the dtype of the weights")
    _check(labels.dim() == 1 and labels.size(0) == hidden.size(0), "one label per row required")
    _check(labels.dtype == torch.int64, "Label type should be CUDA Long")
    _check(int(chunk_rows) > 0, "chunk_rows must be positive")


def _chunks(n, chunk_rows):
    return [(r0, min(n, r0 + chunk_rows)) for r0 in range(0, n, chunk_rows)]


def _chunk_buffer(rows, v, like):
    """[rows, v] view of a buffer whose row pitch is v rounded up to 64 elements."""
    pitch = (v + 63) // 64 * 64
    return torch.empty(rows, pitch, dtype=like.dtype, device=like.device)[:, :v]


def _slice_columns(n, v, chunk_rows):
    """Columns per vocabulary slice of the backward: a [n, columns] buffer as large as the forward's [chunk_rows, v]
    one, in whole groups of 64 columns."""
    return max(64, (min(n, chunk_rows) * ((v + 63) // 64 * 64) // n) // 64 * 64)


def _logits(hidden, weight, bias, r0, r1, buf):
    return linear_gemm.gemm(hidden[r0:r1], weight, trans_b=True, bias=bias, out=buf[:r1 - r0])


class LinearSoftmaxCrossEntropy(torch.autograd.Function):
    """apply(hidden [N, E], weight [V, E], bias [V] | None, labels [N], smoothing=0.0, padding_idx=-100,
    chunk_rows=4096, keep_logits_bytes=16 GiB) -> losses fp32 [N] (zeros where labels == padding_idx): what
    SoftmaxCrossEntropyLoss.apply(F.linear(hidden, weight, bias), labels, smoothing, padding_idx, True) returns."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, labels, smoothing=0.0, padding_idx=-100, chunk_rows=DEFAULT_CHUNK_ROWS,
                keep_logits_bytes=DEFAULT_KEEP_LOGITS_BYTES):
        _check_inputs(hidden, weight, bias, labels, chunk_rows)
        hidden, weight, labels = hidden.contiguous(), weight.contiguous(), labels.contiguous()
        bias = bias.contiguous() if bias is not None else None
        n, v = hidden.size(0), weight.size(0)
        losses = torch.empty(n, dtype=torch.float32, device=hidden.device)
        lse = torch.empty(n, dtype=torch.float32, device=hidden.device)
        ctx.kept = None
        if n > 0:
            _check(v > 0, "Number of classes in input should not be 0")
            pitch = (v + 63) // 64 * 64
            keep = any(ctx.needs_input_grad[:3]) and n * pitch * hidden.element_size() <= int(keep_logits_bytes)
            if keep:
                # the columns between V and the pitch are multiplied by nothing, but the contraction over the classes
                # reads whole 16-byte groups: keep them finite
                full = torch.empty(n, pitch, dtype=hidden.dtype, device=hidden.device)
                full[:, v:].zero_()
                z = linear_gemm.gemm(hidden, weight, trans_b=True, bias=bias, out=full[:, :v])
                part, m = xentropy_cuda.forward(z, labels, smoothing, True, padding_idx=padding_idx)
                losses.copy_(part)
                lse.copy_(m)
                ctx.kept = full
            else:
                buf = _chunk_buffer(min(n, chunk_rows), v, hidden)
                for r0, r1 in _chunks(n, chunk_rows):
                    z = _logits(hidden, weight, bias, r0, r1, buf)
                    part, m = xentropy_cuda.forward(z, labels[r0:r1], smoothing, True, padding_idx=padding_idx)
                    losses[r0:r1] = part
                    lse[r0:r1] = m
        ctx.save_for_backward(hidden, weight, bias, labels, lse)
        ctx.smoothing, ctx.padding_idx, ctx.chunk_rows = smoothing, padding_idx, chunk_rows
        return losses

    @staticmethod
    def _backward_from_kept(ctx, full, grad_loss, hidden, weight, bias, labels, lse, need_h, need_w, need_b):
        """The kept logits become their gradient in place; one contraction with the states, one with the weights."""
        n, v = hidden.size(0), weight.size(0)
        z = full[:, :v]
        dz = xentropy_cuda.backward(grad_loss, z, lse, labels, ctx.smoothing, padding_idx=ctx.padding_idx, out=z)
        dh = dw = db = None
        if need_w:
            dw = linear_gemm.gemm(dz, hidden, trans_a=True)                          # [V, N] x [N, E]
        if need_b:
            db = linear_gemm.colsum(dz)                                              # fixed-order fp32 column sums
        if need_h:
            # the contraction over the classes in whole 64-class steps (the matrix-core loop fed from LDS directly), and
            # the last V % 64 classes as a product of their own; summed in fp32
            v0 = v // 64 * 64
            if v0 == v or v0 == 0:
                dh = linear_gemm.gemm(dz, weight)
            else:
                dh32 = linear_gemm.gemm(full[:, :v0], weight[:v0]).float()
                dh32.add_(linear_gemm.gemm(full[:, v0:v], weight[v0:]))
                dh = dh32.to(hidden.dtype)
        return dh, dw, db

    @staticmethod
    def backward(ctx, grad_loss):
        hidden, weight, bias, labels, lse = ctx.saved_tensors
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_b = bias is not None and ctx.needs_input_grad[2]
        n, v = hidden.size(0), weight.size(0)
        grad_loss = grad_loss.contiguous().float()
        dh = dw = db = None
        if need_w:
            dw = torch.empty_like(weight) if n > 0 else torch.zeros_like(weight)
        if need_b:
            db = torch.empty_like(bias) if n > 0 else torch.zeros_like(bias)
        if need_h:
            dh = torch.empty_like(hidden)
        full, ctx.kept = ctx.kept, None              # consumed below: a second backward recomputes
        if full is not None and n > 0 and (need_h or need_w or need_b):
            dh, dw, db = LinearSoftmaxCrossEntropy._backward_from_kept(ctx, full, grad_loss, hidden, weight, bias, labels, lse,
                                                                       need_h, need_w, need_b)
            return dh, dw, db, None, None, None, None, None
        if n > 0 and (need_h or need_w or need_b):
            # Given the log-sum-exp of each row the logits gradient is elementwise, so the backward walks the
            # vocabulary in slices of whole columns: a slice's weight and bias gradients are complete (contracted over
            # all rows at once, written once) and only the small [N, E] gradient of the states is summed over slices.
            cols = _slice_columns(n, v, ctx.chunk_rows)
            buf = _chunk_buffer(n, min(v, cols), hidden)
            gbuf = _chunk_buffer(n, min(v, cols), hidden)
            dh32 = None
            for c0 in range(0, v, cols):
                c1 = min(v, c0 + cols)
                w_c = weight[c0:c1]
                z = linear_gemm.gemm(hidden, w_c, trans_b=True, bias=None if bias is None else bias[c0:c1],
                                     out=buf[:, :c1 - c0])                           # the forward's logits again
                dz = xentropy_cuda.backward(grad_loss, z, lse, labels, ctx.smoothing, padding_idx=ctx.padding_idx,
                                            out=gbuf[:, :c1 - c0], class_offset=c0, total_classes=v)
                if need_w:
                    linear_gemm.gemm(dz, hidden, trans_a=True, out=dw[c0:c1])        # [V_c, N] x [N, E]
                if need_b:
                    if db.dtype == dz.dtype:
                        linear_gemm.colsum(dz, out=db[c0:c1])                        # fixed-order fp32 column sums
                    else:
                        db[c0:c1] = linear_gemm.colsum(dz)
                if need_h:
                    part = linear_gemm.gemm(dz, w_c)                                 # [N, V_c] x [V_c, E]
                    if c0 == 0 and c1 == v:
                        dh = part
                    elif dh32 is None:
                        dh32 = part.float()
                    else:
                        dh32.add_(part)
            if need_h and dh32 is not None:
                dh.copy_(dh32)
        return dh, dw, db, None, None, None, None, None


def linear_cross_entropy_eval(hidden, weight, bias, labels, padding_idx=-100, chunk_rows=DEFAULT_CHUNK_ROWS):
    """No-gradient pass for validation: -> (losses fp32 [N] without smoothing, argmax int64 [N]); the reference's
    eval branch takes the argmax of the unnormalised logits (onmt/modules/loss.py:293-299)."""
    _check_inputs(hidden, weight, bias, labels, chunk_rows)
    with torch.no_grad():
        hidden, weight, labels = hidden.contiguous(), weight.contiguous(), labels.contiguous()
        bias = bias.contiguous() if bias is not None else None
        n, v = hidden.size(0), weight.size(0)
        losses = torch.empty(n, dtype=torch.float32, device=hidden.device)
        preds = torch.empty(n, dtype=torch.int64, device=hidden.device)
        if n > 0:
            _check(v > 0, "Number of classes in input should not be 0")
            buf = _chunk_buffer(min(n, chunk_rows), v, hidden)
            for r0, r1 in _chunks(n, chunk_rows):
                z = _logits(hidden, weight, bias, r0, r1, buf)
                part, _, best = xentropy_cuda.forward(z, labels[r0:r1], 0.0, True, padding_idx=padding_idx, want_argmax=True)
                losses[r0:r1] = part
                preds[r0:r1] = best          # from the loss kernel's own pass over the row: the chunk is not read again
    return losses, preds


class GeneratorLoss(nn.Module):
    """The reference's Generator (its parameter is `linear`, so checkpoints map key by key) and the fast branch of
    CrossEntropyLossBase._compute_loss in one module.

    forward(hidden [..., E], targets [...], loss_weights=None, loss_constraint=0, sum_loss=True, eval=False)
    -> dict(loss, data, correct, total). `loss` is sum_i w_i (loss_i - loss_constraint) (or the per-row tensor when
    sum_loss is False); `data` is the unweighted, unconstrained sum as a Python float (per-row tensor when sum_loss is
    False), as the reference reports it; label smoothing applies in training mode only. Rows whose target is the
    padding index contribute zero loss and zero gradient (the reference drops them with index_select first);
    `total` counts the others and `correct` (eval=True only) how many of those the argmax hits."""

    def __init__(self, hidden_size, output_size, label_smoothing=0.0, padding_idx=0, bias=True,
                 chunk_rows=DEFAULT_CHUNK_ROWS):
        super().__init__()
        self.linear = nn.Linear(hidden_size, output_size, bias=bias)
        stdv = 1.0 / hidden_size ** 0.5
        nn.init.uniform_(self.linear.weight, -stdv, stdv)
        if bias:
            nn.init.zeros_(self.linear.bias)
        self.hidden_size, self.output_size = hidden_size, output_size
        self.label_smoothing, self.padding_idx, self.chunk_rows = label_smoothing, padding_idx, chunk_rows

    def forward(self, hidden, targets, loss_weights=None, loss_constraint=0, sum_loss=True, eval=False):
        h = hidden.reshape(-1, hidden.size(-1))
        y = targets.reshape(-1)
        correct, total = 0, 0
        if eval:
            rows, preds = linear_cross_entropy_eval(h, self.linear.weight, self.linear.bias, y, self.padding_idx,
                                                    self.chunk_rows)
            real = y != self.padding_idx
            correct, total = int(((preds == y) & real).sum().item()), int(real.sum().item())
        else:
            smoothing = self.label_smoothing if self.training else 0.0
            rows = LinearSoftmaxCrossEntropy.apply(h, self.linear.weight, self.linear.bias, y, smoothing,
                                                   self.padding_idx, self.chunk_rows)
        data = rows.detach().sum().item() if sum_loss else rows.detach()
        # the constraint is subtracted on real rows only: padded rows are not part of the reference's batch
        loss = rows - loss_constraint * (y != self.padding_idx).to(rows.dtype) if loss_constraint else rows
        if loss_weights is not None:
            loss = loss * loss_weights.reshape(-1).to(loss.dtype)
        if sum_loss:
            loss = loss.sum()
        return dict(loss=loss, data=data, correct=correct, total=total)
