"""The benchmark workloads at their full sizes.

Where the CPU oracle cannot run the whole workload in seconds, parity is checked on the slices
that are independent (attention: batch columns; cross-entropy: rows) and the rest through
size-independent properties: probability rows sum to one, exact zeros on masked keys / padded
rows, gradient rows sum to zero, determinism. (The MLP and LayerNorm workloads run whole against
the oracle in test_mlp_gpu.py / test_layer_norm_gpu.py.) The packed-attention and relative-position
workloads are also held against a second, independent computation of the whole batch: fp32 matrix
products on the device, and the chain of separate kernels.
"""
import pytest
import torch

from nmtgminor_amd.native import (encdec_multihead_attn_bias_blaslt as ed, flash_attn_cuda, relative_self_attn_blaslt as rel,
                                  self_multihead_attn_blaslt as sa, xentropy_cuda)
from oracle import attention as oat, flash_attention as ofa, inputs, relative_attention as orel, xentropy as oxe
from util import assert_close

pytestmark = pytest.mark.gpu
D = torch.float64
BF = torch.bfloat16


def test_self_attention_workload(dev):
    T, B, E, H = 512, 32, 1024, 16
    d = inputs.self_attn_inputs(T, B, E, H)                      # seed 1003, bf16, p = 0.1
    g = lambda k: d[k].to(dev)
    lin, scores, dropped, dmask, ctx, out = sa.forward(False, True, H, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"),
                                                        g("pad_mask"), 0.1, dropout_mask=g("dropout_mask"))
    grads = sa.backward(False, H, g("dout"), ctx, dropped, scores, lin, g("x"), g("w_in"), g("w_out"), dmask, 0.1)
    # parity on two batch columns (first, last): every op up to dx is independent per column
    for col in (0, B - 1):
        x1 = d["x"][:, col:col + 1]
        dm1 = d["dropout_mask"].view(B, H, T, T)[col].reshape(H, T, T)
        f = oat.self_attn_fwd(x1, d["w_in"], d["w_out"], d["b_in"], d["b_out"], H, d["pad_mask"][col:col + 1], None, 0.1, dm1,
                              D, round_to=BF)
        bw = oat.self_attn_bwd(d["dout"][:, col:col + 1], x1, d["w_in"], d["w_out"], H, f, 0.1, dm1, D, round_to=BF)
        assert_close(out[:, col:col + 1], f["outputs"], BF, f"outputs[{col}]")
        assert_close(dropped.view(B, H, T, T)[col], f["dropout_results"], BF, f"dropout_results[{col}]")
        assert_close(grads[0][:, col:col + 1], bw["dx"], BF, f"dx[{col}]", scale_atol=True)
    # properties over the whole tensors
    pad = d["pad_mask"].to(dev)
    cov = dropped.view(B, H, T, T)
    assert (cov.permute(0, 3, 1, 2)[pad] == 0).all()                               # masked keys: exactly zero
    assert (cov[g("dropout_mask").view(B, H, T, T) == 0] == 0).all()               # dropped entries: exactly zero
    sc = scores.view(B, H, T, T)
    assert torch.isinf(sc.permute(0, 3, 1, 2)[pad]).all() and torch.isfinite(sc.permute(0, 3, 1, 2)[~pad]).all()
    again = sa.backward(False, H, g("dout"), ctx, dropped, scores, lin, g("x"), g("w_in"), g("w_out"), dmask, 0.1)
    assert all(torch.equal(a, b) for a, b in zip(grads, again))                    # deterministic
    # weight gradients: they are sums over all tokens of products this test already pinned per column; check them
    # against an fp32 product of the library's own per-token gradient and input
    dlin = sa.backward_compact(False, H, torch.matmul(g("dout").view(-1, E).float(), g("w_out").float()).to(BF).view(T, B, E),
                               dropped, scores, lin, dmask, 0.1)[0]
    want = dlin.view(-1, 3 * E).float().t() @ g("x").view(-1, E).float()
    assert_close(grads[1], want.cpu(), BF, "dW_in", scale_atol=True)
    assert_close(grads[3], dlin.view(-1, 3 * E).float().sum(0).cpu(), BF, "db_in", scale_atol=True)


def test_self_attention_workload_weight_gradients_against_the_oracle(dev):
    """Weight and bias gradients sum over every token, so no single batch column pins them. A fixed sub-batch of four
    columns of the workload (full length, width and head count; its own HIP call) is small enough for the fp64 oracle:
    every gradient of that call is compared with it."""
    T, B, E, H = 512, 32, 1024, 16
    d = inputs.self_attn_inputs(T, B, E, H)
    cols = torch.tensor([0, 1, B - 2, B - 1])
    x, dout, pad = d["x"][:, cols].contiguous(), d["dout"][:, cols].contiguous(), d["pad_mask"][cols].contiguous()
    dm = d["dropout_mask"].view(B, H, T, T)[cols].reshape(len(cols) * H, T, T).contiguous()
    g = lambda t: t.to(dev)
    lin, scores, dropped, dmask, ctx, out = sa.forward(False, True, H, g(x), g(d["w_in"]), g(d["w_out"]), g(d["b_in"]),
                                                        g(d["b_out"]), g(pad), 0.1, dropout_mask=g(dm))
    grads = sa.backward(False, H, g(dout), ctx, dropped, scores, lin, g(x), g(d["w_in"]), g(d["w_out"]), dmask, 0.1)
    f = oat.self_attn_fwd(x, d["w_in"], d["w_out"], d["b_in"], d["b_out"], H, pad, None, 0.1, dm, D, round_to=BF)
    bw = oat.self_attn_bwd(dout, x, d["w_in"], d["w_out"], H, f, 0.1, dm, D, round_to=BF)
    assert_close(out, f["outputs"], BF, "outputs")
    assert_close(grads[0], bw["dx"], BF, "dx", scale_atol=True)
    assert_close(grads[1], bw["dw_in"], BF, "dW_in", scale_atol=True)
    assert_close(grads[2], bw["dw_out"], BF, "dW_out", scale_atol=True)
    assert_close(grads[3], bw["db_in"], BF, "db_in", scale_atol=True)
    assert_close(grads[4], bw["db_out"], BF, "db_out", scale_atol=True)


def test_self_attention_workload_without_coverage(dev):
    """The same workload through self_attn_func(return_coverage=False): the tiled core over the padded batch, against the
    oracle in its core="tiled" mode (16-bit roundings where the tiled kernels have them) at the tolerance of every other
    16-bit comparison. Output and input gradient of two batch columns of the full call (every op up to dx is independent
    per column); every gradient, weights and biases included, of a call on a fixed sub-batch of four columns (full length,
    width and head count) that the fp64 oracle can follow; the full call's weight gradients against the extension path's
    on the same inputs as a check of the sums over all 16384 tokens (two 16-bit results of the same sums: relative error
    of the whole tensor); and a second run must repeat the first bit for bit."""
    from nmtgminor_amd.modules.self_attention_func import self_attn_func
    from util import rel_err
    T, B, E, H = 512, 32, 1024, 16
    d = inputs.self_attn_inputs(T, B, E, H)
    names = ("x", "w_in", "w_out", "b_in", "b_out")

    def run(cols=None):
        sub = dict(d)
        if cols is not None:
            sub["x"], sub["dout"] = d["x"][:, cols].contiguous(), d["dout"][:, cols].contiguous()
            sub["pad_mask"] = d["pad_mask"][cols].contiguous()
            sub["dropout_mask"] = d["dropout_mask"].view(B, H, T, T)[cols].reshape(len(cols) * H, T, T).contiguous()
        leaves = [sub[k].to(dev).requires_grad_() for k in names]
        out, cov = self_attn_func(False, True, H, *leaves, sub["pad_mask"].to(dev), 0.1, False, None, False, None, True, False,
                                  False, sub["dropout_mask"].to(dev))
        assert cov.numel() == 0
        out.backward(sub["dout"].to(dev))
        return [out.detach()] + [z.grad for z in leaves], sub

    def oracle(sub):
        f = oat.self_attn_fwd(sub["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], H, sub["pad_mask"], None, 0.1,
                              sub["dropout_mask"], D, round_to=BF, core="tiled")
        return f, oat.self_attn_bwd(sub["dout"], sub["x"], d["w_in"], d["w_out"], H, f, 0.1, sub["dropout_mask"], D, round_to=BF,
                                    core="tiled")

    got, _ = run()
    for col in (0, B - 1):
        one = dict(x=d["x"][:, col:col + 1], dout=d["dout"][:, col:col + 1], pad_mask=d["pad_mask"][col:col + 1],
                   dropout_mask=d["dropout_mask"].view(B, H, T, T)[col].reshape(H, T, T))
        f, bw = oracle(one)
        assert_close(got[0][:, col:col + 1], f["outputs"], BF, f"outputs[{col}]")
        assert_close(got[1][:, col:col + 1], bw["dx"], BF, f"dx[{col}]", scale_atol=True)
    part, sub = run(torch.tensor([0, 1, B - 2, B - 1]))
    f, bw = oracle(sub)
    assert_close(part[0], f["outputs"], BF, "sub-batch outputs")
    for i, key in enumerate(("dx", "dw_in", "dw_out", "db_in", "db_out")):
        assert_close(part[1 + i], bw[key], BF, "sub-batch " + key, scale_atol=True)
    g = lambda k: d[k].to(dev)
    lin, scores, dropped, dmask, ctx, out = sa.forward(False, True, H, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"),
                                                        g("pad_mask"), 0.1, dropout_mask=g("dropout_mask"))
    ext = sa.backward(False, H, g("dout"), ctx, dropped, scores, lin, g("x"), g("w_in"), g("w_out"), dmask, 0.1)
    for i, what in ((1, "dW_in"), (2, "dW_out"), (3, "db_in"), (4, "db_out")):
        assert rel_err(got[1 + i], ext[i].float().cpu()) < 5e-3, what
    again, _ = run()
    assert all(torch.equal(a, b) for a, b in zip(got, again))


def test_decoder_attention_workload(dev):
    TQ, TK, B, E, H = 128, 1500, 16, 1024, 16
    d = inputs.encdec_attn_inputs(TQ, TK, B, E, H)               # seed 1004, bf16, eval
    g = lambda k: d[k].to(dev)
    r = ed.forward(False, H, g("x_q"), g("x_kv"), g("w_q"), g("w_kv"), g("w_out"), g("b_q"), g("b_kv"), g("b_out"),
                   g("pad_mask"), 0.0)
    q_lin, kv_lin, scores, dropped, dmask, ctx, out = r
    assert dmask.numel() == 0 and dropped.shape == (B * H, TQ, TK)
    for col in (0, B - 1):
        f = oat.encdec_attn_fwd(d["x_q"][:, col:col + 1], d["x_kv"][:, col:col + 1], d["w_q"], d["w_kv"], d["w_out"], d["b_q"],
                                d["b_kv"], d["b_out"], H, d["pad_mask"][col:col + 1], 0.0, None, D, round_to=BF)
        assert_close(out[:, col:col + 1], f["outputs"], BF, f"cross outputs[{col}]")
        assert_close(dropped.view(B, H, TQ, TK)[col], f["dropout_results"], BF, f"cross probabilities[{col}]")
    pad = d["pad_mask"].to(dev)
    cov = dropped.view(B, H, TQ, TK)
    assert (cov.permute(0, 3, 1, 2)[pad] == 0).all()
    assert (cov.float().sum(-1) - 1).abs().max() < 2e-2                            # rows sum to one
    # companion causal self-attention, T = 128
    s = inputs.self_attn_inputs(TQ, B, E, H, p=0.0, seed=1004, causal=True)
    gs = lambda k: s[k].to(dev)
    rs = sa.forward(True, False, H, gs("x"), gs("w_in"), gs("w_out"), gs("b_in"), gs("b_out"), gs("time_mask"), 0.0)
    f = oat.self_attn_fwd(s["x"][:, :2], s["w_in"], s["w_out"], s["b_in"], s["b_out"], H, None, s["time_mask"], 0.0, None, D,
                          round_to=BF)
    assert_close(rs[5][:, :2], f["outputs"], BF, "causal self outputs")
    upper = torch.triu(torch.ones(TQ, TQ, device=dev), 1).bool()
    assert (rs[2][:, upper] == 0).all()                                            # no attention to the future


def test_xentropy_workload(dev):
    N, V = 16384, 250054
    d = inputs.xentropy_inputs(N, V, with_logits=False)          # seed 1005 targets, 10 % padding
    gen = torch.Generator(device=dev)
    gen.manual_seed(1005)
    logits = torch.empty(N, V, dtype=BF, device=dev)
    for r0 in range(0, N, 1024):
        logits[r0:r0 + 1024] = (2.0 * torch.randn(1024, V, generator=gen, device=dev)).to(BF)
    labels = d["labels"].to(dev)
    losses, lse = xentropy_cuda.forward(logits, labels, 0.1, True, padding_idx=1)
    grad = xentropy_cuda.backward(d["grad_loss"].to(dev), logits, lse, labels, 0.1, padding_idx=1)
    assert grad.shape == (N, V) and grad.dtype == BF and logits.numel() > 2 ** 31
    # rows are independent: oracle on a sample that covers all four 16-byte row phases and the last row
    rows = torch.tensor([0, 1, 2, 3, 4097, 8190, 12345, N - 2, N - 1])
    lo, lseo = oxe.xentropy_fwd(logits[rows.to(dev)].cpu(), d["labels"][rows], 0.1, 1, D)
    assert_close(losses[rows.to(dev)], lo, torch.float32, "losses", rtol=2e-5, atol=2e-5)
    assert_close(lse[rows.to(dev)], lseo, torch.float32, "lse", rtol=2e-6, atol=2e-5)
    go = oxe.xentropy_bwd(torch.ones(len(rows)), logits[rows.to(dev)].cpu(), lseo, d["labels"][rows], 0.1, 1, D)
    assert_close(grad[rows.to(dev)], go, BF, "dlogits")
    # whole-tensor properties
    pad = labels == 1
    assert int(pad.sum()) >= round(N * 0.1)      # the seeded 10 % plus the Zipf draws that land on index 1
    assert (losses[pad] == 0).all()                                                # bit-exact zeros on padding
    assert int(grad[pad].ne(0).sum()) == 0
    assert torch.isfinite(losses).all() and (losses[~pad] > 0).all()
    ref_lse = torch.stack([torch.logsumexp(logits[i:i + 256].float(), 1) for i in range(0, N, 256)]).view(-1)
    assert (lse - ref_lse).abs().max() < 1e-4                                      # against the library routine, all rows
    row_sums = torch.cat([grad[i:i + 256].float().sum(1) for i in range(0, N, 256)])
    assert row_sums[~pad].abs().max() < 5e-2                                       # softmax - target distribution sums to 0
    tgt = grad[torch.arange(N, device=dev)[~pad], labels[~pad]].float()
    assert (tgt < 0).all() and (tgt > -1.0).all()                                  # target logit gradient in (-(1-eps), 0)


def test_packed_attention_workload(dev):
    """The benchmark's packed workload (32 sequences of U[256, 512] tokens, 16 heads of 64, dropout 0.1 drawn on the
    device): two sequences against the oracle, and every sequence against the same arithmetic written with fp32
    matrix products on the device (scores, softmax, the drawn mask with its scale, autograd for the gradients), to the
    tolerances of test_zze_flash_attention_gpu.py (probabilities rounded to bf16 relative to different reference points)."""
    B, H, Dh, p = 32, 16, 64, 0.1
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(256, 513, (B,), generator=g).tolist()
    cu = torch.zeros(B + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.tensor(lens), 0)
    total, mx = int(cu[-1]), max(lens)
    qkv = torch.randn(total, 3, H, Dh, generator=g).to(BF)
    dout = torch.randn(total, H, Dh, generator=g).to(BF)
    qkv_d, dout_d, cu_d = qkv.to(dev), dout.to(dev), cu.to(dev)
    q, k, v = qkv_d[:, 0], qkv_d[:, 1], qkv_d[:, 2]
    scale = Dh ** -0.5
    torch.cuda.manual_seed(77)
    out = torch.full_like(dout_d, float("nan"))
    lse, mask = flash_attn_cuda.fwd(q, k, v, out, cu_d, cu_d, mx, mx, p, scale, False, False, True)
    state = flash_attn_cuda.last_rng
    dqkv = torch.full_like(qkv_d, float("nan"))
    flash_attn_cuda.bwd(dout_d, q, k, v, out, lse, dqkv[:, 0], dqkv[:, 1], dqkv[:, 2], cu_d, cu_d, mx, mx, p, scale, False, False,
                        rng=state)
    assert not torch.isnan(out).any() and not torch.isnan(dqkv).any()
    keep_scale = 256.0 / round(256 * (1 - p))
    p_eff = 1.0 - 1.0 / keep_scale
    kept = sum(float(mask[b, :, :n, :n].float().sum()) for b, n in enumerate(lens)) / sum(H * n * n for n in lens)
    assert abs(kept - 1 / keep_scale) < 1e-3
    atol, gatol = 8e-3 * 2 / (1 - p), 4e-3 / (1 - p)
    # (a) the oracle on the first and the last sequence
    for b in (0, B - 1):
        sl = slice(int(cu[b]), int(cu[b + 1]))
        n = lens[b]
        one = torch.tensor([0, n], dtype=torch.int32)
        m1 = mask[b:b + 1, :, :n, :n].cpu()
        want, _ = ofa.flash_attn_fwd(qkv[sl, 0], qkv[sl, 1], qkv[sl, 2], one, one, n, scale, False, p_eff, m1, D, round_to=BF)
        wdq, wdk, wdv, _ = ofa.flash_attn_bwd(dout[sl], qkv[sl, 0], qkv[sl, 1], qkv[sl, 2], one, one, n, scale, False, p_eff, m1, D,
                                              round_to=BF)
        assert_close(out[sl], want, BF, f"out[{b}]", atol=atol)
        for i, (name, w) in enumerate((("dq", wdq), ("dk", wdk), ("dv", wdv))):
            assert_close(dqkv[sl, i], w, BF, f"{name}[{b}]", scale_atol=True, atol=gatol)
    # (b) every sequence against fp32 matrix products on the device
    for b, n in enumerate(lens):
        sl = slice(int(cu[b]), int(cu[b + 1]))
        x = qkv_d[sl].float().requires_grad_()
        qs, ks, vs = (x[:, i].transpose(0, 1) for i in range(3))                   # [H, n, Dh]
        prob = torch.softmax(qs @ ks.transpose(1, 2) * scale, dim=-1) * mask[b, :, :n, :n].float() * keep_scale
        ref = (prob @ vs).transpose(0, 1)
        ref.backward(dout_d[sl].float())
        assert_close(out[sl], ref.detach().cpu(), BF, f"out of sequence {b}", atol=atol)
        assert_close(lse[b, :, :n], torch.logsumexp(qs.detach() @ ks.detach().transpose(1, 2) * scale, -1).cpu(), torch.float32,
                     f"lse of sequence {b}", rtol=1e-3, atol=2e-3)
        for i, name in enumerate(("dq", "dk", "dv")):
            assert_close(dqkv[sl, i], x.grad[:, i].cpu(), BF, f"{name} of sequence {b}", scale_atol=True, atol=gatol)
    # (c) deterministic, and the backward that refills its own keep bits from the generator state agrees bit for bit
    again = torch.full_like(qkv_d, float("nan"))
    flash_attn_cuda.bwd(dout_d, q, k, v, out, lse, again[:, 0], again[:, 1], again[:, 2], cu_d, cu_d, mx, mx, p, scale, False, False,
                        rng=state[:4])
    assert torch.equal(again, dqkv)


def test_relative_attention_workload(dev, monkeypatch):
    """The benchmark's relative-position workload (T = 512, B = 32, E = 1024, 16 heads, 512 positions): the kernels that run
    the shift inside the softmax against the chain of separate kernels on the whole batch (same rounding points, rows
    added up in another order: four 16-bit units on the probabilities, the usual tolerances behind the products), and
    two batch columns against the oracle."""
    T, B, E, H, p = 512, 32, 1024, 16, 0.1
    names = ("x", "pos", "w_in", "w_out", "w_pos", "b_in", "b_out", "b_pos", "r_w_bias", "r_r_bias")
    d = inputs.rel_self_attn_inputs(T, B, E, H, BF, p=p, seed=1006)
    a = {k: d[k].to(dev) for k in names}
    a["pos"] = a["pos"].repeat(1, B, 1).contiguous()          # one position projection per batch column, as the extension lays it out
    pad, dm, dout = d["pad_mask"].to(dev), d["dropout_mask"].to(dev), d["dout"].to(dev)

    def run():
        res = rel.forward(True, False, H, a["x"], a["pos"], a["w_in"], a["w_out"], a["w_pos"], a["b_in"], a["b_out"], a["b_pos"],
                          a["r_w_bias"], a["r_r_bias"], pad, p, dropout_mask=dm)
        lin, pos_lin, scores, dropped, dmask, ctx, out = res
        grads = rel.backward(H, dout, ctx, dropped, scores, lin, pos_lin, a["r_w_bias"], a["r_r_bias"], a["x"], a["pos"], a["w_in"],
                             a["w_out"], a["w_pos"], dmask, p, pad_mask=pad)
        return scores, dropped, out, grads

    scores, dropped, out, grads = run()
    monkeypatch.setenv("NMTG_REL_FUSED", "0")
    scores0, dropped0, out0, grads0 = run()
    monkeypatch.delenv("NMTG_REL_FUSED")
    assert torch.equal(scores, scores0)                                   # the summed scores: same additions, same rounding
    ulp4 = 4 * torch.finfo(BF).eps
    torch.testing.assert_close(dropped.float(), dropped0.float(), rtol=ulp4, atol=1e-4 * ulp4)
    assert_close(out, out0.cpu(), BF, "outputs, fused against separate")
    for i, (x, y) in enumerate(zip(grads, grads0)):
        assert_close(x, y.cpu(), BF, f"gradient {i}, fused against separate", scale_atol=True)
    cov = dropped.view(B, H, T, T)
    assert (cov.permute(0, 3, 1, 2)[pad] == 0).all() and (cov[dm.view(B, H, T, T) == 0] == 0).all()
    # two batch columns against the oracle (every result but the weight gradients is independent per column)
    for col in (0, B - 1):
        sub = {k: (d[k][:, col:col + 1] if k == "x" else d[k]) for k in names}      # the positions are shared by the columns
        dm1 = d["dropout_mask"].view(B, H, T, T)[col].reshape(H, T, T)
        f = orel.rel_self_attn_fwd(*(sub[k] for k in names), H, d["pad_mask"][col:col + 1], None, p, dm1, D, round_to=BF)
        g = orel.rel_self_attn_bwd(d["dout"][:, col:col + 1], sub["x"], sub["pos"], d["w_in"], d["w_out"], d["w_pos"], H, f, p, dm1, D,
                                   round_to=BF)
        assert_close(out[:, col:col + 1], f["outputs"], BF, f"outputs[{col}]", flips=2e-3)
        assert_close(cov[col], f["dropout_results"], BF, f"dropout_results[{col}]")
        assert_close(grads[0][:, col:col + 1], g["dx"], BF, f"dx[{col}]", scale_atol=True)


def test_products_with_operands_beyond_four_gib(dev):
    """Operands of 4.6 and 4.9 GB through the GEMM entry point: the matrix-core loop fed from LDS directly addresses an
    operand from its tile's first row, so its 32-bit lane offsets hold whatever the operand's size. Row blocks from the
    start, the 4 GiB boundary and the end of each result against fp64 on those rows."""
    from nmtgminor_amd.native import linear_gemm
    g = torch.Generator(device=dev)
    g.manual_seed(77)
    m, k, n = 70000, 32768, 128
    a = torch.randn(m, k, generator=g, device=dev, dtype=torch.bfloat16)           # rows of 64 KiB: 4 GiB ends at row 65536
    b = (torch.randn(n, k, generator=g, device=dev) / k ** 0.5).to(torch.bfloat16)
    c = linear_gemm.gemm(a, b, trans_b=True)
    for r0 in (0, 65400, m - 256):
        want = a[r0:r0 + 256].double() @ b.double().t()
        assert_close(c[r0:r0 + 256], want.cpu(), torch.bfloat16, f"C = A B^T, rows from {r0}", scale_atol=True)
    del a, c
    kk, mm = 8192, 300000                                                          # A^T B with A [K, M]: rows of 600 KB
    at = torch.randn(kk, mm, generator=g, device=dev, dtype=torch.bfloat16)
    bt = (torch.randn(kk, n, generator=g, device=dev) / kk ** 0.5).to(torch.bfloat16)
    ct = linear_gemm.gemm(at, bt, trans_a=True)
    assert ct.shape == (mm, n)
    for c0 in (0, 150000, mm - 256):
        want = at[:, c0:c0 + 256].double().t() @ bt.double()
        assert_close(ct[c0:c0 + 256], want.cpu(), torch.bfloat16, f"C = A^T B, rows from {c0}", scale_atol=True)


def test_projection_and_loss_workload(dev):
    """The benchmark's projection + loss (16384 positions x 1024 -> 250054 classes, eps 0.1, padding index 1) with the
    logits kept once (8.2 GB) and without them (rows in chunks forward, class slices recomputed backward). Losses and the
    gradient of the states on sampled rows (rows are independent given the weights), the weight gradient on sampled
    classes (a class's row of it is a sum over all positions of that class's logit gradients, which the oracle forms
    from the fp64 logits of that class and the log-sum-exp checked on the sampled rows), zeros on padding, and the two
    memory policies against each other."""
    from nmtgminor_amd.modules.generator_loss import LinearSoftmaxCrossEntropy
    N, E, V, eps, pad_idx = 16384, 1024, 250054, 0.1, 1
    d = inputs.xentropy_inputs(N, V, with_logits=False)
    labels, gl = d["labels"], d["grad_loss"]
    g = torch.Generator(device=dev)
    g.manual_seed(1006)
    h = torch.randn(N, E, generator=g, device=dev).to(BF)
    w = (torch.randn(V, E, generator=g, device=dev) / E ** 0.5).to(BF)

    def run(budget):
        hd, wd = h.clone().requires_grad_(), w.clone().requires_grad_()
        losses = LinearSoftmaxCrossEntropy.apply(hd, wd, None, labels.to(dev), eps, pad_idx, 4096, budget)
        losses.backward(gl.to(dev))
        return losses.detach(), hd.grad, wd.grad

    kept = run(16 << 30)
    rows = torch.tensor([0, 1, 4097, 12345, N - 1])
    rows = rows[labels[rows] != pad_idx] if (labels[rows] != pad_idx).any() else rows
    hc, wc = h.cpu(), w.cpu()
    z = (hc[rows].to(D) @ wc.to(D).t()).to(BF)                                   # the logits as stored
    lo, lseo = oxe.xentropy_fwd(z, labels[rows], eps, pad_idx, D)
    assert_close(kept[0][rows.to(dev)], lo, BF, "losses", atol=2e-3)
    dz = oxe.xentropy_bwd(gl[rows], z, lseo, labels[rows], eps, pad_idx, D).to(BF).to(D)
    assert_close(kept[1][rows.to(dev)], dz @ wc.to(D), BF, "gradient of the states, sampled rows")
    # sampled classes: the most frequent target, a rare one, the last class
    classes = torch.tensor([int(labels[labels != pad_idx].mode().values), 7, V - 1])
    zc = (hc.to(D) @ wc[classes].to(D).t()).to(BF).to(D)                         # [N, 3]
    # per-row log-sum-exp over all classes, from the device's logits of the kept run's twin: recompute it in slices
    lse = torch.empty(N, dtype=torch.float64)
    for r0 in range(0, N, 2048):
        zz = (h[r0:r0 + 2048].float() @ w.float().t()).to(BF).float()
        lse[r0:r0 + 2048] = torch.logsumexp(zz, 1).double().cpu()
    assert (lse[rows] - lseo).abs().max() < 2e-3
    real = (labels != pad_idx).to(D)
    p = torch.exp(zc - lse[:, None])
    target = (labels[:, None] == classes[None, :]).to(D)
    dzc = ((p - eps / V - (1 - eps) * target) * (gl.to(D) * real)[:, None]).to(BF).to(D)
    assert_close(kept[2][classes.to(dev)], dzc.t() @ hc.to(D), BF, "weight gradient, sampled classes", scale_atol=True)
    pad = (labels == pad_idx).to(dev)
    assert (kept[0][pad] == 0).all() and int(kept[1][pad].ne(0).sum()) == 0
    assert torch.isfinite(kept[2]).all()
    lean = run(0)
    assert_close(lean[0], kept[0].cpu(), BF, "losses, the two memory policies", atol=2e-3)
    assert_close(lean[1], kept[1].float().cpu(), BF, "gradient of the states, the two memory policies")
    from util import rel_err
    assert rel_err(lean[2], kept[2].float().cpu()) < 5e-3
