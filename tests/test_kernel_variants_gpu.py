"""Pairs of code paths that compute the same thing: the default one and the plainer one that the library falls back to
for shapes the default does not take, forced here by its switch (NAME=0 in the environment, read on every call):

  NMTG_ATTN_FUSED=0    Q K^T -> mask, then softmax -> dropout as two kernels instead of one (rows of up to 512 keys)
  NMTG_GEMM_SKINNY=0   a product with at most 32 rows against a row-major weight on the tiled kernels instead of the
                       kernel that gives every wavefront one output column
  NMTG_ATTN_DECODE=0   a one-position decoding step as one-row batched GEMMs and a softmax instead of the kernel that
                       streams the cached keys and values once

Each of those tests runs both paths in one process and compares them with each other and the default one with the CPU
oracle. The other tests here hold single-path kernels with a special form (the 256x64 ring tile, the gelu table, padded
keys, the MLP backward's one reduction launch) to the oracle.
"""
import os

import pytest
import torch

from nmtgminor_amd.native import encdec_multihead_attn_bias_blaslt as ed_native, fused_mlp_gelu, self_multihead_attn_blaslt as sa_native
from nmtgminor_amd.native.linear_gemm import gemm
from oracle import attention as oat, inputs, mlp as omlp
from util import assert_close

pytestmark = pytest.mark.gpu
D = torch.float64


class off:
    """NAME=0 inside the block, the previous setting afterwards."""

    def __init__(self, name):
        self.name = name

    def __enter__(self):
        self.before = os.environ.get(self.name)
        os.environ[self.name] = "0"

    def __exit__(self, *exc):
        if self.before is None:
            os.environ.pop(self.name, None)
        else:
            os.environ[self.name] = self.before


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch,m,n,k", [(8, 512, 64, 512), (3, 300, 64, 192), (2, 256, 64, 64), (5, 77, 64, 128)])
def test_ring_256x64_products(dev, dtype, batch, m, n, k):
    """The 256x64 tile of the slot-ring loop (the per-head products P V, dS K, Pd^T dC, dS^T Q) against fp64."""
    g = torch.Generator().manual_seed(91)
    a = torch.randn(batch, m, k, generator=g).to(dtype).to(dev)
    b_kn = torch.randn(batch, k, n, generator=g).to(dtype).to(dev)        # NN: P V, dS K
    a_km = torch.randn(batch, k, m, generator=g).to(dtype).to(dev)        # TN: Pd^T dC, dS^T Q
    got_nn = gemm(a, b_kn)
    got_tn = gemm(a_km, b_kn, trans_a=True, split_k=False)
    assert_close(got_nn, a.double().cpu() @ b_kn.double().cpu(), dtype, "nn", scale_atol=True)
    assert_close(got_tn, a_km.double().cpu().transpose(1, 2) @ b_kn.double().cpu(), dtype, "tn", scale_atol=True)


def _self_fwd(dev, d, h, p, fused):
    g = lambda k: d[k].to(dev) if d[k] is not None else None
    dm = g("dropout_mask") if p > 0 else None
    mask = g("time_mask") if d["time_mask"] is not None else g("pad_mask")
    args = (d["time_mask"] is not None, True, h, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), mask, p)
    if not fused:
        with off("NMTG_ATTN_FUSED"):
            return sa_native.forward(*args, dropout_mask=dm)
    return sa_native.forward(*args, dropout_mask=dm)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("t,b,e,h,p,causal", [(512, 2, 256, 4, 0.1, False), (128, 3, 512, 8, 0.0, False),
                                              (200, 2, 256, 4, 0.25, False), (96, 2, 128, 2, 0.1, True),
                                              (40, 2, 128, 2, 0.1, False)])
def test_fused_scores_softmax_matches_two_kernel_path(dev, dtype, t, b, e, h, p, causal):
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=p, seed=92, causal=causal, zero_bias=False)
    lin0, sc0, dr0, dm0, ctx0, out0 = _self_fwd(dev, d, h, p, fused=False)
    lin1, sc1, dr1, dm1, ctx1, out1 = _self_fwd(dev, d, h, p, fused=True)
    assert torch.equal(lin0, lin1)
    assert torch.equal(sc0, sc1)                         # scores: same product, same rounding, same -inf pattern
    assert_close(dr1.float(), dr0.float().cpu(), dtype, "dropped vs two-kernel path")
    assert torch.equal(dr1 == 0, dr0 == 0)               # masked keys and dropped units: zeros in the same places
    fwd = oat.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], d["time_mask"], p,
                            d["dropout_mask"] if p > 0 else None, D, round_to=dtype)
    assert_close(dr1, fwd["dropout_results"], dtype, "dropped vs oracle")
    assert_close(out1, fwd["outputs"], dtype, "outputs vs oracle")


def test_fused_scores_softmax_rng_mask_is_the_same_stream(dev):
    # Philox keep-mask keyed by (seed, offset, element index): both paths must draw the same mask
    dtype = torch.bfloat16
    t, b, e, h = 64, 2, 128, 2
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=0.0, seed=93, zero_bias=False)
    g = lambda k: d[k].to(dev)
    args = (False, True, h, g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out"), g("pad_mask"), 0.3)
    torch.cuda.manual_seed(17)
    with off("NMTG_ATTN_FUSED"):
        r0 = sa_native.forward(*args)
    torch.cuda.manual_seed(17)
    r1 = sa_native.forward(*args)
    assert torch.equal(r0[3], r1[3])
    assert_close(r1[2].float(), r0[2].float().cpu(), dtype, "dropped (rng)")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("t,b,e,h,p,causal", [(512, 2, 256, 4, 0.1, False), (200, 2, 256, 4, 0.25, False),
                                              (96, 2, 128, 2, 0.0, True), (40, 2, 128, 2, 0.1, False)])
def test_fused_softmax_backward_matches_two_kernel_path(dev, dtype, t, b, e, h, p, causal):
    d = inputs.self_attn_inputs(t, b, e, h, dtype, p=p, seed=94, causal=causal, zero_bias=False)
    lin, scores, dropped, dmask, ctx, out = _self_fwd(dev, d, h, p, fused=False)
    g = lambda k: d[k].to(dev)
    args = (causal, h, g("dout"), ctx, dropped, scores, lin, g("x"), g("w_in"), g("w_out"), dmask, p)
    with off("NMTG_ATTN_FUSED"):
        ref = sa_native.backward(*args)
    got = sa_native.backward(*args)
    fwd = oat.self_attn_fwd(d["x"], d["w_in"], d["w_out"], d["b_in"], d["b_out"], h, d["pad_mask"], d["time_mask"], p,
                            d["dropout_mask"] if p > 0 else None, D, round_to=dtype)
    bwd = oat.self_attn_bwd(d["dout"], d["x"], d["w_in"], d["w_out"], h, fwd, p, d["dropout_mask"] if p > 0 else None, D,
                            round_to=dtype)
    for name, a_, r_, o_ in zip(("dx", "dw_in", "dw_out", "db_in", "db_out"), got, ref,
                                (bwd["dx"], bwd["dw_in"], bwd["dw_out"], bwd["db_in"], bwd["db_out"])):
        assert_close(a_, r_.float().cpu(), dtype, name + " vs two-kernel path", scale_atol=True)
        assert_close(a_, o_, dtype, name + " vs oracle", scale_atol=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tokens,dm,di,p", [(256, 128, 256, 0.1), (300, 192, 448, 0.0), (128, 512, 2048, 0.2)])
def test_table_gelu_matches_the_formula(dev, dtype, tokens, dm, di, p):
    """The ring kernels' activation epilogues read Phi from a 2049-entry table in LDS. From the pre-activations the kernel
    stored, the formula in fp64 gives what the post-activations should be: the table's are the same 16-bit numbers nearly
    everywhere and one unit in the last place apart elsewhere."""
    # wide pre-activations (|h| up to ~8): both ends of the table and the clamp beyond them are used
    d = inputs.mlp_inputs(tokens, dm, di, dtype, p=p, seed=95, zero_bias=False)
    d["x"] = (d["x"].float() * 4).to(dtype)
    ins = [d[k].to(dev) for k in ("x", "w1", "w2", "b1", "b2")]
    ins[0].requires_grad_()                                      # asks the backward for dx
    mask = d["mask"].to(dev) if p > 0 else None
    dy = d["dy"].to(dev)
    got = fused_mlp_gelu.forward(p, ins, mask)
    ggot = fused_mlp_gelu.backward(p, dy, got, ins)
    pre = got[2].double().cpu().view(tokens, di)
    assert pre.abs().max() > 6.5 and (pre.abs() < 0.05).any()
    post = omlp.act_fwd(pre, "gelu") * (d["mask"].double() / (1.0 - p) if p > 0 else 1.0)
    post16 = post.to(dtype)
    stored = got[1].view(tokens, di)
    same = (stored.cpu() == post16).float().mean().item()
    assert same > 0.9, same           # the differing ones sit in the negative tail, where gelu itself is below 1e-2
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7      # largest relative size of one unit in the last place
    assert_close(stored, post16.double(), dtype, "post-activations: table vs formula", rtol=1.05 * ulp, atol=3e-5)
    ws, bs = [d["w1"], d["w2"]], [d["b1"], d["b2"]]
    masks = [d["mask"]] if p > 0 else None
    y, pre_o, post_o = omlp.mlp_fwd(d["x"], ws, bs, "gelu", p, masks, D, round_to=dtype)
    gx, gws, gbs = omlp.mlp_bwd(d["dy"], d["x"], ws, pre_o, post_o, "gelu", p, masks, D, round_to=dtype)
    assert_close(got[0], y, dtype, "y vs oracle", scale_atol=True)
    assert_close(ggot[0], gx, dtype, "dx vs oracle", scale_atol=True)
    assert_close(ggot[1], gws[0], dtype, "dW1 vs oracle", scale_atol=True)
    assert_close(ggot[2], gws[1], dtype, "dW2 vs oracle", scale_atol=True)
    assert_close(ggot[3], gbs[0], dtype, "db1 vs oracle", scale_atol=True)
    assert_close(ggot[4], gbs[1], dtype, "db2 vs oracle", scale_atol=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tq,tk,b,e,h,masked", [(17, 100, 3, 128, 2, True), (32, 1500, 2, 256, 4, True), (8, 70, 2, 128, 2, False)])
def test_padded_keys_give_the_same_cross_attention(dev, dtype, tq, tk, b, e, h, masked):
    """Inference cross-attention with a key length that is not a multiple of 64 runs on keys / values padded with masked
    zero rows (every tensor of the middle section 16-byte aligned); what comes back are views of the true length."""
    d = inputs.encdec_attn_inputs(tq, tk, b, e, h, dtype, p=0.0, seed=96, zero_bias=False)
    g = lambda k: d[k].to(dev) if d[k] is not None else None
    pad = g("pad_mask") if masked else None
    got = ed_native.forward(False, h, g("x_q"), g("x_kv"), g("w_q"), g("w_kv"), g("w_out"), g("b_q"), g("b_kv"), g("b_out"), pad, 0.0)
    assert got[2].shape == (b * h, tq, tk) and not got[2].is_contiguous()      # views of the padded rows
    fwd = oat.encdec_attn_fwd(d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], d["b_q"], d["b_kv"], d["b_out"], h,
                              d["pad_mask"] if masked else None, 0.0, None, D, round_to=dtype)
    assert_close(got[0], fwd["input_lin_q_results"], dtype, "q projection")
    assert_close(got[1], fwd["input_lin_kv_results"], dtype, "kv projection")
    assert_close(got[6], fwd["outputs"], dtype, "outputs vs oracle")
    assert_close(got[3], fwd["dropout_results"], dtype, "probabilities vs oracle")
    if masked:
        assert (got[3].view(b, h, tq, tk).permute(0, 3, 1, 2)[g("pad_mask")] == 0).all()    # masked keys: exactly 0
    # the backward accepts the views (it copies them into the layout its kernels read)
    grads = ed_native.backward(h, g("dout"), got[5], got[3], got[2], got[0], got[1], g("x_q"), g("x_kv"), g("w_q"), g("w_kv"),
                               g("w_out"), None, 0.0)
    bwd = oat.encdec_attn_bwd(d["dout"], d["x_q"], d["x_kv"], d["w_q"], d["w_kv"], d["w_out"], h, fwd, 0.0, None, D, round_to=dtype)
    for a_, key in zip(grads, ("dx_q", "dx_kv", "dw_q", "dw_kv", "dw_out", "db_q", "db_kv", "db_out")):
        assert_close(a_, bwd[key], dtype, key + " from the views", scale_atol=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tokens,dm,di", [(4096, 128, 256), (1000, 192, 448), (8192, 512, 2048)])
def test_mlp_backward_with_one_reduction_launch(dev, dtype, tokens, dm, di):
    """Split-K reductions and bias-gradient sums of all layers are jobs of one reduction (riding with the last
    data-gradient product, or a launch at the end): shapes that split K and shapes that do not, against the oracle; the
    input-gradient-only backward must give the same dx bit for bit."""
    p = 0.1
    d = inputs.mlp_inputs(tokens, dm, di, dtype, p=p, seed=98, zero_bias=False)
    ins = [d[k].to(dev) for k in ("x", "w1", "w2", "b1", "b2")]
    ins[0].requires_grad_()
    mask, dy = d["mask"].to(dev), d["dy"].to(dev)
    out = fused_mlp_gelu.forward(p, ins, mask)
    got = fused_mlp_gelu.backward(p, dy, out, ins)
    only_dx = fused_mlp_gelu.backward_input_only(p, dy, out, ins)
    assert torch.equal(only_dx[0], got[0])
    ws = [d["w1"], d["w2"]]
    gx, gws, gbs = omlp.mlp_bwd(d["dy"], d["x"], ws, [out[2].cpu().view(tokens, di)], [out[1].cpu().view(tokens, di)], "gelu", p, [d["mask"]], D, round_to=dtype)
    for a_, w_, name in zip(got, [gx] + gws + gbs, ("dx", "dW1", "dW2", "db1", "db2")):
        assert_close(a_, w_, dtype, name, scale_atol=True)


def test_three_layer_mlp_backward_with_one_reduction_launch(dev):
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(99)
    tokens, sizes = 2048, (96, 320, 160, 64)
    x = torch.randn(tokens, sizes[0], generator=g).to(dtype)
    ws = [(0.05 * torch.randn(sizes[i + 1], sizes[i], generator=g)).to(dtype) for i in range(3)]
    bs = [(0.1 * torch.randn(sizes[i + 1], generator=g)).to(dtype) for i in range(3)]
    dy = torch.randn(tokens, sizes[-1], generator=g).to(dtype)
    ins = [x.to(dev).requires_grad_()] + [w.to(dev) for w in ws] + [b_.to(dev) for b_ in bs]
    out = fused_mlp_gelu.forward(0.0, ins)
    got = fused_mlp_gelu.backward(0.0, dy.to(dev), out, ins)
    assert len(got) == 7
    y, pre_o, post_o = omlp.mlp_fwd(x, ws, bs, "gelu", 0.0, None, D, round_to=dtype)
    gx, gws, gbs = omlp.mlp_bwd(dy, x, ws, pre_o, post_o, "gelu", 0.0, None, D, round_to=dtype)
    for a_, w_, name in zip(got, [gx] + gws + gbs, ("dx", "dW1", "dW2", "dW3", "db1", "db2", "db3")):
        assert_close(a_, w_, dtype, name, scale_atol=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tk,b,e,h,masked", [(1500, 3, 256, 4, True), (127, 2, 128, 4, False), (70, 2, 256, 2, True),
                                             (300, 2, 256, 8, True), (1, 1, 128, 2, False)])
def test_decode_step_kernel_matches_the_gemm_path_and_the_oracle(dev, dtype, tk, b, e, h, masked):
    from nmtgminor_amd.modules import incremental as inc
    g = torch.Generator().manual_seed(tk + e)
    q = torch.randn(1, b, e, generator=g).to(dtype)
    keys = torch.randn(tk, b, e, generator=g).to(dtype)
    values = torch.randn(tk, b, e, generator=g).to(dtype)
    pad = None
    if masked:
        lengths = torch.randint(max(1, tk // 2), tk + 1, (b,), generator=g)
        lengths[0] = 0 if tk > 1 else 1                                   # a sentence without any live key: zeros
        pad = torch.arange(tk).view(1, tk) >= lengths.view(b, 1)
    args = (h, q.to(dev), keys.to(dev), values.to(dev), None if pad is None else pad.to(dev))
    ctx, probs = inc._core(*args)
    with off("NMTG_ATTN_DECODE"):
        ctx_g, probs_g = inc._core(*args)
    d = e // h
    qh, kh, vh = (t.to(D).view(-1, b * h, d).transpose(0, 1) for t in (q, keys, values))          # [B*H, T, D]
    sc = (qh @ kh.transpose(1, 2) * d ** -0.5).to(dtype).to(D)                                    # stored in 16 bits
    if pad is not None:
        sc = sc.masked_fill(pad.repeat_interleave(h, 0).view(b * h, 1, tk), float("-inf"))
    want_p = torch.nan_to_num(torch.softmax(sc, -1), nan=0.0).to(dtype).to(D)
    want_c = (want_p @ vh).transpose(0, 1).reshape(1, b, e)
    assert probs.shape == (b * h, 1, tk) and ctx.shape == (1, b, e)
    assert_close(probs, want_p, dtype, "probabilities")
    assert_close(ctx, want_c, dtype, "context", atol=2e-3)
    assert_close(probs, probs_g.cpu(), dtype, "probabilities, both paths")
    assert_close(ctx, ctx_g.cpu(), dtype, "context, both paths", atol=2e-3)
    if masked and tk > 1:
        assert float(probs[:h].abs().max()) == 0.0 and float(ctx[:, 0].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(32, 1024, 1024), (1, 256, 64), (7, 100, 2056), (32, 64, 8), (20, 1000, 3000), (32, 4096, 1024)])
def test_few_row_products_match_the_tiled_kernels(dev, dtype, m, n, k):
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).to(dtype).to(dev)
    w = (torch.randn(n, k, generator=g) * k ** -0.5).to(dtype).to(dev)
    bias = torch.randn(n, generator=g).to(dtype).to(dev)
    got = gemm(x, w, False, True, alpha=0.5, bias=bias)
    with off("NMTG_GEMM_SKINNY"):
        tiled = gemm(x, w, False, True, alpha=0.5, bias=bias)
    want = 0.5 * (x.double() @ w.double().t()).cpu() + bias.double().cpu()
    assert_close(got, want, dtype, "few-row kernel")
    assert_close(tiled, want, dtype, "tiled")
    pitched = torch.full((m, k + 24), float("nan"), dtype=dtype, device=dev)      # rows with a pitch, NaN in the padding
    pitched[:, :k] = x
    assert torch.equal(gemm(pitched[:, :k], w, False, True, alpha=0.5, bias=bias), got)
