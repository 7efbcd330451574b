"""Thin Python face of nmtg_gemm: row-major strided-batched products on the MFMA units.
Used by the tests and by callers that need a plain projection (the reference's linear_blaslt,
onmt/modules/extensions/mlp_blaslt/linear.cpp:142-144)."""
import torch

from .. import _lib as L


def gemm(a, b, trans_a=False, trans_b=False, alpha=1.0, bias=None, out=None, split_k=True):
    """a: [.., m, k] (or [.., k, m] if trans_a); b: [.., k, n] (or [.., n, k] if trans_b); the
    last two dims may be strided views as long as the innermost stride is 1 and the batch is a
    single leading dim with a uniform stride. Returns [.., m, n] in the input dtype."""
    L.require_cuda(a, b, bias, out)
    if a.dim() == 2:
        a3, b3 = a.unsqueeze(0), b.unsqueeze(0)
    else:
        a3, b3 = a, b
    if a3.dim() != 3 or b3.dim() != 3 or a3.shape[0] != b3.shape[0]:
        raise RuntimeError("gemm: operands must be [batch, rows, cols] with equal batch")
    if a3.stride(2) != 1 or b3.stride(2) != 1:
        raise RuntimeError("gemm: innermost stride must be 1")
    if a3.dtype != b3.dtype or a3.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise RuntimeError("gemm: fp32, fp16 or bf16 operands of one dtype required")
    batch = a3.shape[0]
    m, k = (a3.shape[2], a3.shape[1]) if trans_a else (a3.shape[1], a3.shape[2])
    kb, n = (b3.shape[2], b3.shape[1]) if trans_b else (b3.shape[1], b3.shape[2])
    if k != kb:
        raise RuntimeError("gemm: inner dimensions differ")
    if out is None:
        out = torch.empty(batch, m, n, dtype=a3.dtype, device=a3.device)
    o3 = out if out.dim() == 3 else out.unsqueeze(0)
    if k == 0 and o3.numel() > 0:          # an empty sum: alpha * 0 (+ bias)
        o3.zero_()
        if bias is not None:
            o3.add_(bias)
        return out if a.dim() == 3 else o3[0]
    ws = None
    ws_bytes = 0
    if split_k and trans_a and not trans_b and a3.dtype != torch.float32:      # the fp32 kernel never splits K
        ws_bytes = int(L.load().nmtg_gemm_workspace_bytes(L.i64(m), L.i64(n), L.i64(k), L.i64(batch)))
        if ws_bytes:
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a3.device)
    L.call("nmtg_gemm", L.i32(int(trans_a)), L.i32(int(trans_b)), L.i64(m), L.i64(n), L.i64(k), L.f32(alpha),
           L.ptr(a3), L.i64(a3.stride(1)), L.i64(a3.stride(0)), L.ptr(b3), L.i64(b3.stride(1)), L.i64(b3.stride(0)),
           L.ptr(o3), L.i64(o3.stride(1)), L.i64(o3.stride(0)), L.i64(batch), L.ptr(bias), L.ptr(ws), L.i64(ws_bytes),
           L.i32(L.dtype_code(a3)), L.stream_of(a3))
    return out if a.dim() == 3 else o3[0]


def colsum(x, out=None):
    """x [rows, cols] (row-major, innermost stride 1, any row pitch) -> sum over the rows, [cols] in x's dtype, fp32
    accumulation in a fixed order (the reference's torch.sum(grads, 0) behind every bias gradient)."""
    L.require_cuda(x, out)
    if x.dim() != 2 or (x.size(1) > 1 and x.stride(1) != 1):
        raise RuntimeError("colsum: a [rows, cols] matrix with unit innermost stride required")
    rows, cols = x.shape
    if out is None:
        out = torch.empty(cols, dtype=x.dtype, device=x.device)
    elif out.shape != (cols,) or out.dtype != x.dtype or not out.is_contiguous():
        raise RuntimeError("colsum: out must be a contiguous [cols] tensor of the input dtype")
    if rows == 0:
        return out.zero_()
    if cols == 0:
        return out
    ws_bytes = int(L.load().nmtg_colsum_workspace_bytes(L.i64(rows), L.i64(cols)))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    L.call("nmtg_colsum", L.ptr(x), L.i64(rows), L.i64(cols), L.i64(x.stride(0) if rows > 1 else max(cols, x.stride(0))),
           L.ptr(out), L.ptr(ws), L.i64(ws_bytes), L.i32(L.dtype_code(x)), L.stream_of(x))
    return out
