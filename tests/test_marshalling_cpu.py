"""Every Python stand-in hands the C ABI exactly what include/nmtg_hip.h declares.

ctypes calls are positional and untyped: a missing, extra or mis-typed argument would corrupt the
call silently. Here `_lib.call` is replaced by a recorder that checks, for every entry point the
stand-ins reach, the argument count and each argument's ctypes class against the parameter list
parsed from the header (pointer -> c_void_p / ctypes array / None, int64_t -> c_int64, uint64_t ->
c_uint64, int -> c_int, float -> c_float). No kernel runs; the tensors live on the CPU and the
device checks of the stand-ins are switched off for the test.
"""
import ctypes
import re

import pytest
import torch

from nmtgminor_amd import _lib, _rng
from nmtgminor_amd.native import (encdec_multihead_attn_bias_blaslt as ed, fast_layer_norm_cuda as ln,
                                  fused_dropout_add_cuda as da, fused_mlp_agelu, fused_mlp_gelu, fused_mlp_relu,
                                  fused_mlp_silu, fused_optim, linear_blaslt, linear_gemm, mask_softmax_dropout_cuda as sm, mlp_gelu_blaslt,
                                  relative_position,                                  self_multihead_attn_blaslt as sa, xentropy_cuda as xe)


def header_signatures():
    with open(_lib.HEADER_PATH) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    sigs = {}
    for m in re.finditer(r"\b(?:int|int64_t|const char\*)\s+(nmtg_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        params = [p.strip() for p in m.group(2).split(",")]
        if params == ["void"]:
            params = []
        kinds = []
        for p in params:
            if "*" in p:
                kinds.append("ptr")
            elif re.match(r"(const\s+)?int64_t\b", p):
                kinds.append("i64")
            elif re.match(r"(const\s+)?uint64_t\b", p):
                kinds.append("u64")
            elif re.match(r"(const\s+)?float\b", p):
                kinds.append("f32")
            elif re.match(r"(const\s+)?int\b", p):
                kinds.append("i32")
            else:
                raise AssertionError(f"unrecognised parameter '{p}' of {m.group(1)}")
        sigs[m.group(1)] = kinds
    return sigs


SIGS = header_signatures()


def kind_of(arg):
    if arg is None or isinstance(arg, (ctypes.c_void_p, ctypes.c_char_p, ctypes.Array)) or isinstance(arg, ctypes._Pointer):
        return "ptr"
    if isinstance(arg, ctypes.c_int64):
        return "i64"
    if isinstance(arg, ctypes.c_uint64):
        return "u64"
    if isinstance(arg, ctypes.c_float):
        return "f32"
    if isinstance(arg, ctypes.c_int):
        return "i32"
    return f"unsupported {type(arg).__name__}"


@pytest.fixture
def recorder(monkeypatch):
    calls = []

    def fake_call(name, *args):
        assert name in SIGS, f"{name} is not declared in the header"
        got = [kind_of(a) for a in args]
        assert got == SIGS[name], f"{name}: passes {got}, header declares {SIGS[name]}"
        calls.append(name)

    monkeypatch.setattr(_lib, "call", fake_call)
    monkeypatch.setattr(_lib, "require_cuda", lambda *t: None)
    monkeypatch.setattr(_lib, "stream_of", lambda t: ctypes.c_void_p(0))
    for mod in (ed, sa, sm, da):
        for attr in ("philox_seed_offset",):
            if hasattr(mod, attr):
                monkeypatch.setattr(mod, attr, lambda dev, n: (123, 0))
    import nmtgminor_amd.native._mlp_common as mc
    import nmtgminor_amd.native._attn_common as ac
    for mod in (mc, ac):
        if hasattr(mod, "philox_seed_offset"):
            monkeypatch.setattr(mod, "philox_seed_offset", lambda dev, n: (123, 0))
    monkeypatch.setattr(_rng, "philox_seed_offset", lambda dev, n: (123, 0))
    return calls


def test_header_is_parsed_completely():
    assert set(SIGS) == set(_lib.header_functions())
    assert SIGS["nmtg_version"] == [] and SIGS["nmtg_ln_fwd"][:6] == ["ptr"] * 6


BF = torch.bfloat16


def test_layer_norm_and_elementwise(recorder):
    x = torch.randn(6, 32)
    g, b = torch.ones(32), torch.zeros(32)
    z, mu, rs = ln.ln_fwd(x, g, b, 1e-5)
    ln.ln_bwd(torch.randn(6, 32), x, mu, rs, g, None, False)
    ln.ln_bwd(torch.randn(6, 32), z, None, rs, g, b, True)
    mask = torch.ones(40, dtype=torch.uint8)
    m, out = da.forward(True, torch.randn(40), torch.randn(40), 0.1, mask)
    da.forward(True, torch.randn(40), torch.randn(40), 0.1)            # mask drawn by the kernel
    da.forward(False, torch.randn(40), torch.randn(40), 0.1)
    da.backward(torch.randn(40), m, 0.1)
    s = torch.randn(4, 5, 16)
    pad = torch.zeros(2, 16, dtype=torch.bool)
    dm = torch.ones(4, 5, 16, dtype=torch.uint8)
    _, p_, d_ = sm.forward(True, 2, s, 0.1, pad_mask=pad, dropout_mask=dm)
    sm.forward(True, 2, s, 0.1)
    sm.forward(False, 2, s, 0.0, time_mask=torch.zeros(5, 16, dtype=torch.bool))
    sm.backward(2, torch.randn(4, 5, 16), p_, dm, 0.1)
    sm.backward_recompute(2, torch.randn(4, 5, 16), None, s, dm, 0.1, pad_mask=pad)
    logits = torch.randn(7, 19)
    labels = torch.zeros(7, dtype=torch.int64)
    losses, lse = xe.forward(logits, labels, 0.1, False, padding_idx=1)
    xe.forward(logits.to(BF), labels, 0.1, True)
    xe.backward(torch.ones(7), logits, lse, labels, 0.1, padding_idx=1)
    assert {"nmtg_ln_fwd", "nmtg_ln_bwd", "nmtg_dropout_add_fwd", "nmtg_dropout_add_bwd", "nmtg_softmax_dropout_fwd",
            "nmtg_softmax_dropout_bwd", "nmtg_xentropy_fwd", "nmtg_xentropy_bwd"} <= set(recorder)


def test_mlp_and_gemm(recorder):
    x = torch.randn(8, 16).to(BF)
    w1, w2 = torch.randn(32, 16).to(BF), torch.randn(16, 32).to(BF)
    b1, b2 = torch.zeros(32).to(BF), torch.zeros(16).to(BF)
    ins = [x, w1, w2, b1, b2]
    mask = torch.ones(8 * 32, dtype=torch.uint8)
    dy = torch.randn(8, 16).to(BF)
    for mod in (fused_mlp_gelu, fused_mlp_silu, fused_mlp_agelu):
        out = mod.forward(0.1, ins, mask)
        mod.backward(0.1, dy, out, ins)
        mod.forward(0.1, ins)                                          # mask drawn by the kernel
        mod.forward(0.0, ins)
    o = fused_mlp_relu.forward(0.1, False, ins, mask)
    fused_mlp_relu.backward(0.1, dy, o, ins)
    o = fused_mlp_relu.forward(0.1, True, ins, mask)
    fused_mlp_relu.backward_recompute(0.1, dy, o[2], ins)
    out = mlp_gelu_blaslt.forward(0.1, ins, mask)
    mlp_gelu_blaslt.backward(0.1, False, dy, out, ins)
    mlp_gelu_blaslt.backward(0.1, True, dy, (out[0], out[-1]), ins)
    mlp_gelu_blaslt.backward_input_only(0.1, dy, out, ins)
    # three layers, no biases on the middle one
    w3 = torch.randn(8, 16).to(BF)
    fused_mlp_gelu.forward(0.0, [x, w1, w2, w3, b1, b2, torch.zeros(8).to(BF)])
    linear_gemm.gemm(x, w1, False, True)
    linear_gemm.gemm(torch.randn(3, 8, 16).to(BF), torch.randn(3, 16, 24).to(BF))
    linear_gemm.gemm(torch.randn(16, 8).to(BF), torch.randn(16, 24).to(BF), trans_a=True)
    assert {"nmtg_mlp_fwd", "nmtg_mlp_bwd", "nmtg_gemm"} <= set(recorder)


def test_attention(recorder):
    t, tk, b, e, h = 6, 9, 2, 32, 2
    r = lambda *s: torch.randn(*s).to(BF)
    x, w_in, w_out, b_in, b_out = r(t, b, e), r(3 * e, e), r(e, e), r(3 * e), r(e)
    pad = torch.zeros(b, t, dtype=torch.bool)
    dm = torch.ones(b * h, t, t, dtype=torch.uint8)
    lin, scores, dropped, dmask, ctx, out = sa.forward(False, True, h, x, w_in, w_out, b_in, b_out, pad, 0.1, dropout_mask=dm)
    sa.forward(False, True, h, x, w_in, w_out, None, None, pad, 0.1)                   # no biases, kernel-drawn mask
    sa.forward(True, False, h, x, w_in, w_out, b_in, b_out, torch.zeros(t, t, dtype=torch.bool), 0.0)
    sa.backward(False, h, r(t, b, e), ctx, dropped, scores, lin, x, w_in, w_out, dmask, 0.1)
    sa.backward_input_only(False, h, r(t, b, e), ctx, dropped, scores, lin, x, w_in, w_out, dmask, 0.1)
    sa.forward_compact(False, True, h, lin, pad, 0.1, dropout_mask=dm)
    sa.backward_compact(False, h, r(t, b, e), dropped, scores, lin, dmask, 0.1)
    sa.backward_recompute(False, h, r(t, b, e), x, w_in, w_out, b_in, b_out, pad, dm, 0.1)
    x_kv, w_q, w_kv, b_q, b_kv = r(tk, b, e), r(e, e), r(2 * e, e), r(e), r(2 * e)
    padk = torch.zeros(b, tk, dtype=torch.bool)
    dmk = torch.ones(b * h, t, tk, dtype=torch.uint8)
    res = ed.forward(True, h, x, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, padk, 0.1, dropout_mask=dmk)
    q_lin, kv_lin, sc, dr, dmask2, ctx2, out2 = res
    ed.forward(True, h, x, x_kv, w_q, w_kv, w_out, None, None, None, padk, 0.1)
    ed.backward(h, r(t, b, e), ctx2, dr, sc, q_lin, kv_lin, x, x_kv, w_q, w_kv, w_out, dmask2, 0.1)
    ed.backward_input_only(h, r(t, b, e), ctx2, dr, sc, q_lin, kv_lin, x, x_kv, w_q, w_kv, w_out, dmask2, 0.1)
    ed.forward_compact(True, h, q_lin, kv_lin, padk, 0.1, dropout_mask=dmk)
    ed.backward_compact(h, r(t, b, e), dr, sc, q_lin, kv_lin, dmask2, 0.1)
    ed.backward_recompute(h, r(t, b, e), x, x_kv, w_q, w_kv, b_q, b_kv, w_out, dmask2, padk, 0.1)
    assert {"nmtg_self_attn_fwd", "nmtg_self_attn_bwd", "nmtg_encdec_attn_fwd", "nmtg_encdec_attn_bwd"} <= set(recorder)


def test_relative_position_column_sums_and_linear_layer(recorder):
    r = lambda *s: torch.randn(*s).to(BF)
    lin = r(5, 6, 3, 16)
    relative_position.query_bias(lin[:, :, 0, :], r(2, 16), r(2, 16), 2)
    relative_position.shift_add_(r(6, 5, 5), r(6, 5, 8))
    relative_position.shift_backward(r(6, 5, 5), 8)
    relative_position.add_rows(r(6, 5, 8), r(6, 5, 8))
    relative_position.add_rows(r(6, 5, 8), r(6, 5, 3, 8)[:, :, 1, :], out=r(6, 5, 3, 8)[:, :, 0, :])
    linear_gemm.colsum(r(40, 24))
    linear_gemm.colsum(r(40, 32)[:, :24], out=torch.empty(24).to(BF))
    linear_blaslt.forward(r(4, 3, 16), r(24, 16), r(24))
    linear_blaslt.backward(r(4, 3, 16), r(24, 16), r(4, 3, 24), True)
    assert {"nmtg_rel_query_bias", "nmtg_rel_shift_add", "nmtg_rel_shift_bwd", "nmtg_add_rows", "nmtg_colsum",
            "nmtg_gemm"} <= set(recorder)


def test_multi_tensor_optimizer_passes(recorder):
    t = lambda n=12: torch.zeros(n)
    fused_optim.multi_tensor_adam(65536, None, [[t(), t(5)], [t(), t(5)], [t(), t(5)], [t(), t(5)]], 1e-3, 0.9, 0.99, 1e-8, 1, 1, 1, 0.0)
    fused_optim.multi_tensor_scale(65536, torch.zeros(1, dtype=torch.int32), [[t().to(BF)], [t()]], 0.5)
    fused_optim.multi_tensor_scale(65536, None, [[t()], [t()]], 0.5)
    fused_optim.multi_tensor_l2norm(65536, None, [[t(), t(0), t(70000)]], True)
    fused_optim.multi_tensor_axpby(65536, torch.zeros(1, dtype=torch.int32), [[t().to(BF)], [t()], [t()]], 1.0, 2.0, -1)
    fused_optim.multi_tensor_l2norm_scale(65536, None, [[t()], [t().to(BF)]], 0.5, True)
    assert {"nmtg_multi_tensor_adam", "nmtg_multi_tensor_scale", "nmtg_multi_tensor_l2norm", "nmtg_multi_tensor_axpby",
            "nmtg_multi_tensor_l2norm_scale"} <= set(recorder)
