"""CPU stand-in for libnmtg_hip.so — TEST INFRASTRUCTURE ONLY.

`install(monkeypatch)` replaces `nmtgminor_amd._lib.call` by an emulator that decodes an entry
point's ctypes arguments in the order include/nmtg_hip.h declares them (the tensors live in host
memory), computes the result with the CPU oracle and writes it into the output buffers. It lets the
Python side of the build — the stand-in modules, the autograd Functions and the nn.Modules — run
end to end without a GPU, so that argument order, shapes, aliasing and gradient plumbing are tested
on the CPU. It says nothing about the kernels and is never imported by the product package.
"""
import ctypes

import numpy as np
import torch

from nmtgminor_amd import _lib, _rng
from oracle import attention as oat, dropout_add as oda, layer_norm as oln, mlp as omlp, softmax_dropout as osd, xentropy as oxe

D = torch.float64
DT = {0: torch.float32, 1: torch.float16, 2: torch.bfloat16}
ACTS = {0: "none", 1: "relu", 2: "gelu", 3: "silu", 4: "agelu"}


def v(a):
    return a.value if hasattr(a, "value") else a


def T(ptr, shape, dtype):
    p = v(ptr) if not isinstance(ptr, int) else ptr
    if not p:
        return None
    n = int(np.prod(shape)) if len(shape) else 1
    if n == 0:
        return torch.empty(*shape, dtype=dtype)
    nbytes = n * torch.empty(0, dtype=dtype).element_size()
    buf = (ctypes.c_char * nbytes).from_address(p)
    return torch.frombuffer(buf, dtype=dtype, count=n).view(*shape)


def put(dst, src):
    if dst is not None:
        dst.copy_(src.reshape(dst.shape).to(dst.dtype))


def ln_fwd(x, gamma, beta, z, mu, rsigma, rows, hidden, eps, in_dt, w_dt, st):
    rows, hidden = v(rows), v(hidden)
    X, G, B = T(x, (rows, hidden), DT[v(in_dt)]), T(gamma, (hidden,), DT[v(w_dt)]), T(beta, (hidden,), DT[v(w_dt)])
    zo, muo, rso = oln.ln_fwd(X, G, B, v(eps), D)
    put(T(z, (rows, hidden), DT[v(w_dt)]), zo)
    put(T(mu, (rows,), torch.float32), muo)
    put(T(rsigma, (rows,), torch.float32), rso)


def ln_bwd(dz, xz, mu, rsigma, gamma, beta, dx, dgamma, dbeta, dgp, dbp, n_part, rows, hidden, memeff, in_dt, w_dt, st):
    rows, hidden, n_part = v(rows), v(hidden), v(n_part)
    wd, idt = DT[v(w_dt)], DT[v(in_dt)]
    DZ = T(dz, (rows, hidden), wd)
    G = T(gamma, (hidden,), wd)
    RS = T(rsigma, (rows,), torch.float32)
    if v(memeff):
        Z = T(xz, (rows, hidden), idt)
        dxo, dgo, dbo = oln.ln_bwd_memory_efficient(DZ, Z, RS, G, T(beta, (hidden,), wd), D)
    else:
        X = T(xz, (rows, hidden), idt)
        dxo, dgo, dbo = oln.ln_bwd(DZ, X, T(mu, (rows,), torch.float32), RS, G, D)
    put(T(dx, (rows, hidden), idt), dxo)
    put(T(dgamma, (hidden,), wd), dgo)
    put(T(dbeta, (hidden,), wd), dbo)
    P, Q = T(dgp, (n_part, hidden), torch.float32), T(dbp, (n_part, hidden), torch.float32)
    P.zero_(); Q.zero_()
    P[0] = dgo.float(); Q[0] = dbo.float()


def dropout_add_fwd(x, residual, mask, n, p, mode, seed, offset, dt, st):
    n = v(n)
    X, R = T(x, (n,), DT[v(dt)]), T(residual, (n,), DT[v(dt)])
    mode = v(mode)
    if mode == 0:
        put(X, oda.dropout_add_fwd(X, R, None, 0.0, D))
    else:
        M = T(mask, (n,), torch.uint8)
        if mode == 2:
            M.copy_((torch.rand(n) < 1 - v(p)).to(torch.uint8))
        put(X, oda.dropout_add_fwd(X, R, M, v(p), D))


def dropout_add_bwd(go, mask, gx, n, p, dt, st):
    n = v(n)
    put(T(gx, (n,), DT[v(dt)]), oda.dropout_add_bwd(T(go, (n,), DT[v(dt)]), T(mask, (n,), torch.uint8), v(p), D)[0])


def _kmask(key_mask, kind, rows, cols, q_len, heads):
    kind = v(kind)
    if kind == 1:
        b = rows // (heads * q_len)
        return T(key_mask, (b, cols), torch.uint8).bool(), None
    if kind == 2:
        return None, T(key_mask, (q_len, cols), torch.uint8).bool()
    return None, None


def softmax_fwd(scores, key_mask, kind, sm_out, dr_out, dmask, dmode, p, seed, offset, rows, cols, q_len, heads, dt, st):
    rows, cols, q_len, heads = v(rows), v(cols), v(q_len), v(heads)
    bh = rows // q_len
    S = T(scores, (bh, q_len, cols), DT[v(dt)])
    pad, tm = _kmask(key_mask, kind, rows, cols, q_len, heads)
    masked = osd.masked_scores(S.to(D), pad_mask=pad, time_mask=tm, heads=heads)
    dm = None
    if v(dmode):
        dm = T(dmask, (bh, q_len, cols), torch.uint8)
        if v(dmode) == 2:
            dm.copy_((torch.rand(bh, q_len, cols) < 1 - v(p)).to(torch.uint8))
    sm, dr = osd.softmax_dropout_fwd(masked, dm, v(p) if dm is not None else 0.0, D)
    put(T(sm_out, (bh, q_len, cols), DT[v(dt)]), sm)
    put(T(dr_out, (bh, q_len, cols), DT[v(dt)]), dr)


def softmax_bwd(grad, saved, is_scores, key_mask, kind, dmask, dmode, p, gs, rows, cols, q_len, heads, dt, st):
    rows, cols, q_len, heads = v(rows), v(cols), v(q_len), v(heads)
    bh = rows // q_len
    shape = (bh, q_len, cols)
    G = T(grad, shape, DT[v(dt)]).to(D)
    SV = T(saved, shape, DT[v(dt)]).to(D)
    if v(is_scores):
        pad, tm = _kmask(key_mask, kind, rows, cols, q_len, heads)
        SV, _ = osd.softmax_dropout_fwd(osd.masked_scores(SV, pad_mask=pad, time_mask=tm, heads=heads), None, 0.0, D)
    dm = T(dmask, shape, torch.uint8) if v(dmode) else None
    put(T(gs, shape, DT[v(dt)]), osd.softmax_dropout_bwd(G, SV, dm, v(p) if dm is not None else 0.0, D))


def xent_fwd(logits, labels, losses, lse, rows, vocab, ld, smoothing, pad, dt, st):
    n, vv = v(rows), v(vocab)
    lo, ls = oxe.xentropy_fwd(T(logits, (n, v(ld)), DT[v(dt)])[:, :vv], T(labels, (n,), torch.int64), v(smoothing), v(pad), D)
    put(T(losses, (n,), torch.float32), lo)
    put(T(lse, (n,), torch.float32), ls)


def xent_bwd(gl, logits, lse, labels, gout, rows, vocab, ld, ldg, c0, total, smoothing, pad, dt, st):
    n, vv, c0, total = v(rows), v(vocab), v(c0), v(total)
    # a slice of the classes: embed it in a row of `total` classes (the other columns do not influence the slice)
    z = torch.zeros(n, total, dtype=D)
    z[:, c0:c0 + vv] = T(logits, (n, v(ld)), DT[v(dt)])[:, :vv].to(D)
    g = oxe.xentropy_bwd(T(gl, (n,), torch.float32), z, T(lse, (n,), torch.float32).to(D),
                         T(labels, (n,), torch.int64), v(smoothing), v(pad), D)
    put(T(gout, (n, v(ldg)), DT[v(dt)])[:, :vv], g[:, c0:c0 + vv])


def _ptrs(arr, n):
    return [arr[i] for i in range(n)]


def mlp_fwd(nl, x, weights, biases, out_features, batch, in_f, out, post, pre, mask, mode, p, seed, offset, act, dt, st):
    nl, batch, in_f = v(nl), v(batch), v(in_f)
    dtp = DT[v(dt)]
    outs = [out_features[i] for i in range(nl)]
    ins = [in_f] + outs[:-1]
    W = [T(w, (outs[i], ins[i]), dtp) for i, w in enumerate(_ptrs(weights, nl))]
    Bs = [T(b, (outs[i],), dtp) if b else None for i, b in enumerate(_ptrs(biases, nl))]
    X = T(x, (batch, in_f), dtp)
    hidden = sum(outs[:-1]) * batch
    masks = None
    if v(mode):
        M = T(mask, (hidden,), torch.uint8)
        if v(mode) == 2:
            M.copy_((torch.rand(hidden) < 1 - v(p)).to(torch.uint8))
        masks, off = [], 0
        for o in outs[:-1]:
            masks.append(M[off:off + batch * o].view(batch, o)); off += batch * o
    y, pres, posts = omlp.mlp_fwd(X, W, Bs, ACTS[v(act)], v(p) if masks else 0.0, masks, D, round_to=dtp)
    put(T(out, (batch, outs[-1]), dtp), y)
    if hidden:
        put(T(post, (hidden,), dtp), torch.cat([t.reshape(-1) for t in posts]))
        if v(pre):
            put(T(pre, (hidden,), dtp), torch.cat([t.reshape(-1) for t in pres]))


def mlp_bwd(nl, x, weights, out_features, batch, in_f, grad_out, post, pre, mask, p, act, gx, gws, gbs, ws, wsb, dt, st):
    nl, batch, in_f = v(nl), v(batch), v(in_f)
    dtp = DT[v(dt)]
    outs = [out_features[i] for i in range(nl)]
    ins = [in_f] + outs[:-1]
    W = [T(w, (outs[i], ins[i]), dtp) for i, w in enumerate(_ptrs(weights, nl))]
    X = T(x, (batch, in_f), dtp)
    hidden = sum(outs[:-1]) * batch
    posts, pres, masks, off = [], [], [], 0
    PO = T(post, (hidden,), dtp) if hidden else None
    PR = T(pre, (hidden,), dtp) if (hidden and v(pre)) else None
    M = T(mask, (hidden,), torch.uint8) if (hidden and v(mask)) else None
    for o in outs[:-1]:
        posts.append(PO[off:off + batch * o].view(batch, o).to(D))
        pres.append((PR if PR is not None else PO)[off:off + batch * o].view(batch, o).to(D))
        if M is not None:
            masks.append(M[off:off + batch * o].view(batch, o))
        off += batch * o
    pp = v(p) if M is not None else 0.0
    if PR is None and v(p) > 0 and M is None:      # relu from the dropped output
        masks = [(t > 0).to(torch.uint8) for t in posts]; pp = v(p)
        pres = [torch.ones_like(t) for t in posts]
    dx, dws, dbs = omlp.mlp_bwd(T(grad_out, (batch, outs[-1]), dtp), X, W, pres, posts, ACTS[v(act)], pp,
                                masks if masks else None, D, round_to=dtp)
    put(T(gx, (batch, in_f), dtp), dx)
    for i in range(nl):
        if gws is not None and gws[i]:
            put(T(gws[i], (outs[i], ins[i]), dtp), dws[i])
        if gbs is not None and gbs[i]:
            put(T(gbs[i], (outs[i],), dtp), dbs[i])


def self_attn_fwd(x, w_in, w_out, b_in, b_out, mask, kind, lin, scores, sm_out, dropped, dmask, dmode, p, seed, offset, ctx,
                  out, t, b, e, heads, dt, st):
    t, b, e, h = v(t), v(b), v(e), v(heads)
    dtp = DT[v(dt)]
    pad = T(mask, (b, t), torch.uint8).bool() if v(kind) == 1 else None
    tm = T(mask, (t, t), torch.uint8).bool() if v(kind) == 2 else None
    dm = None
    if v(dmode):
        dm = T(dmask, (b * h, t, t), torch.uint8)
        if v(dmode) == 2:
            dm.copy_((torch.rand(b * h, t, t) < 1 - v(p)).to(torch.uint8))
    pp = v(p) if dm is not None else 0.0
    if not v(x):              # compact form: lin is an input, only the attention core runs
        d = e // h
        L3 = T(lin, (t, b * h, 3, d), dtp).to(D)
        sc, sm, dr, cx = oat._core_fwd(L3[:, :, 0], L3[:, :, 1], L3[:, :, 2], h, pad, tm, pp, dm, D, round_to=dtp)
        f = dict(attn_scores=sc, softmax_results=sm, dropout_results=dr, matmul2_results=cx.reshape(t, b, e))
    else:
        f = oat.self_attn_fwd(T(x, (t, b, e), dtp), T(w_in, (3 * e, e), dtp), T(w_out, (e, e), dtp), T(b_in, (3 * e,), dtp),
                              T(b_out, (e,), dtp), h, pad, tm, pp, dm, D, round_to=dtp)
        put(T(lin, (t, b, 3 * e), dtp), f["input_lin_results"])
        put(T(out, (t, b, e), dtp), f["outputs"])
    put(T(scores, (b * h, t, t), dtp), f["attn_scores"])
    put(T(sm_out, (b * h, t, t), dtp), f["softmax_results"])
    put(T(dropped, (b * h, t, t), dtp), f["dropout_results"])
    put(T(ctx, (t, b, e), dtp), f["matmul2_results"])


def self_attn_bwd(grad_out, ctx, dropped, scores, lin, x, w_in, w_out, dmask, p, gx, gwi, gwo, gbi, gbo, glin, ws, wsb, t, b,
                  e, heads, dt, st):
    t, b, e, h = v(t), v(b), v(e), v(heads)
    dtp = DT[v(dt)]
    S = T(scores, (b * h, t, t), dtp).to(D)
    sm, _ = osd.softmax_dropout_fwd(S, None, 0.0, D)
    dm = T(dmask, (b * h, t, t), torch.uint8) if v(dmask) and v(p) > 0 else None
    C = T(ctx, (t, b, e), dtp)
    X, WI, WO = T(x, (t, b, e), dtp), T(w_in, (3 * e, e), dtp), T(w_out, (e, e), dtp)
    if WO is None:            # compact form: grad_out is the context gradient, only grad_lin is wanted
        WO = torch.eye(e, dtype=dtp)
        X = torch.zeros(t, b, e, dtype=dtp)
        WI = torch.zeros(3 * e, e, dtype=dtp)
        C = torch.zeros(t, b, e, dtype=dtp)
    fwd = dict(matmul2_results=C, input_lin_results=T(lin, (t, b, 3 * e), dtp), softmax_results=sm,
               dropout_results=T(dropped, (b * h, t, t), dtp))
    g = oat.self_attn_bwd(T(grad_out, (t, b, e), dtp), X, WI, WO, h, fwd, v(p) if dm is not None else 0.0, dm, D, round_to=dtp)
    put(T(gx, (t, b, e), dtp), g["dx"])
    put(T(gwi, (3 * e, e), dtp), g["dw_in"])
    put(T(gwo, (e, e), dtp), g["dw_out"])
    put(T(gbi, (3 * e,), dtp), g["db_in"])
    put(T(gbo, (e,), dtp), g["db_out"])
    put(T(glin, (t, b, 3 * e), dtp), g["dlin"])


def encdec_fwd(x_q, x_kv, w_q, w_kv, w_out, b_q, b_kv, b_out, pad_mask, q_lin, kv_lin, scores, sm_out, dropped, dmask, dmode,
               p, seed, offset, ctx, out, tq, tk, b, e, heads, dt, st):
    tq, tk, b, e, h = v(tq), v(tk), v(b), v(e), v(heads)
    dtp = DT[v(dt)]
    pad = T(pad_mask, (b, tk), torch.uint8).bool() if v(pad_mask) else None
    dm = T(dmask, (b * h, tq, tk), torch.uint8) if v(dmode) else None
    pp = v(p) if dm is not None else 0.0
    if not v(x_q):            # compact form: q_lin / kv_lin are inputs
        d = e // h
        Q = T(q_lin, (tq, b * h, d), dtp).to(D)
        KV = T(kv_lin, (tk, b * h, 2, d), dtp).to(D)
        sc, sm, dr, cx = oat._core_fwd(Q, KV[:, :, 0], KV[:, :, 1], h, pad, None, pp, dm, D, round_to=dtp)
        f = dict(attn_scores=sc, softmax_results=sm, dropout_results=dr, matmul2_results=cx.reshape(tq, b, e))
    else:
        f = oat.encdec_attn_fwd(T(x_q, (tq, b, e), dtp), T(x_kv, (tk, b, e), dtp), T(w_q, (e, e), dtp), T(w_kv, (2 * e, e), dtp),
                                T(w_out, (e, e), dtp), T(b_q, (e,), dtp), T(b_kv, (2 * e,), dtp), T(b_out, (e,), dtp), h, pad,
                                pp, dm, D, round_to=dtp)
        put(T(q_lin, (tq, b, e), dtp), f["input_lin_q_results"])
        put(T(kv_lin, (tk, b, 2 * e), dtp), f["input_lin_kv_results"])
        put(T(out, (tq, b, e), dtp), f["outputs"])
    put(T(scores, (b * h, tq, tk), dtp), f["attn_scores"])
    put(T(sm_out, (b * h, tq, tk), dtp), f["softmax_results"])
    put(T(dropped, (b * h, tq, tk), dtp), f["dropout_results"])
    put(T(ctx, (tq, b, e), dtp), f["matmul2_results"])


def encdec_bwd(grad_out, ctx, dropped, scores, q_lin, kv_lin, x_q, x_kv, w_q, w_kv, w_out, dmask, p, gxq, gxkv, gwq, gwkv,
               gwo, gbq, gbkv, gbo, gql, gkvl, ws, wsb, tq, tk, b, e, heads, dt, st):
    tq, tk, b, e, h = v(tq), v(tk), v(b), v(e), v(heads)
    d = e // h
    dtp = DT[v(dt)]
    rnd = lambda t_: t_.to(dtp).to(D)
    S = T(scores, (b * h, tq, tk), dtp).to(D)
    sm, _ = osd.softmax_dropout_fwd(S, None, 0.0, D)
    dm = T(dmask, (b * h, tq, tk), torch.uint8) if v(dmask) and v(p) > 0 else None
    pp = v(p) if dm is not None else 0.0
    Q = T(q_lin, (tq, b * h, d), dtp).to(D)
    KV = T(kv_lin, (tk, b * h, 2, d), dtp).to(D)
    g = T(grad_out, (tq, b, e), dtp).to(D).reshape(tq * b, e)
    WO = T(w_out, (e, e), dtp)
    if WO is not None:        # full form: out-projection gradients, then the context gradient
        C = T(ctx, (tq, b, e), dtp).to(D).reshape(tq * b, e)
        put(T(gwo, (e, e), dtp), g.t() @ C)
        put(T(gbo, (e,), dtp), g.sum(0))
        g = rnd(g @ WO.to(D))
    dq, dk, dv = oat._core_bwd(g.view(tq, b * h, d), Q, KV[:, :, 0], KV[:, :, 1], sm, T(dropped, (b * h, tq, tk), dtp).to(D),
                               pp, dm, D, round_to=dtp)
    dq2 = dq.reshape(tq * b, e)
    dkv2 = torch.stack([dk, dv], dim=2).reshape(tk * b, 2 * e)
    put(T(gql, (tq, b, e), dtp), dq2)
    put(T(gkvl, (tk, b, 2 * e), dtp), dkv2)
    XQ, XKV, WQ, WKV = T(x_q, (tq, b, e), dtp), T(x_kv, (tk, b, e), dtp), T(w_q, (e, e), dtp), T(w_kv, (2 * e, e), dtp)
    if XQ is not None:
        put(T(gxq, (tq, b, e), dtp), dq2 @ WQ.to(D))
        put(T(gwq, (e, e), dtp), dq2.t() @ XQ.to(D).reshape(tq * b, e))
        put(T(gbq, (e,), dtp), dq2.sum(0))
    if XKV is not None:
        put(T(gxkv, (tk, b, e), dtp), dkv2 @ WKV.to(D))
        put(T(gwkv, (2 * e, e), dtp), dkv2.t() @ XKV.to(D).reshape(tk * b, e))
        put(T(gbkv, (2 * e,), dtp), dkv2.sum(0))


EMU = {"nmtg_ln_fwd": ln_fwd, "nmtg_ln_bwd": ln_bwd, "nmtg_dropout_add_fwd": dropout_add_fwd,
       "nmtg_dropout_add_bwd": dropout_add_bwd, "nmtg_softmax_dropout_fwd": softmax_fwd, "nmtg_softmax_dropout_bwd": softmax_bwd,
       "nmtg_xentropy_fwd": xent_fwd, "nmtg_xentropy_bwd": xent_bwd, "nmtg_mlp_fwd": mlp_fwd, "nmtg_mlp_bwd": mlp_bwd,
       "nmtg_self_attn_fwd": self_attn_fwd, "nmtg_self_attn_bwd": self_attn_bwd, "nmtg_encdec_attn_fwd": encdec_fwd, "nmtg_encdec_attn_bwd": encdec_bwd}


def fake_call(name, *args):
    if name not in EMU:
        raise NotImplementedError(f"rehearsal: {name} is not emulated")
    EMU[name](*args)


def install(monkeypatch):
    """Route every C call of the stand-ins to the emulator and switch their device checks off."""
    monkeypatch.setattr(_lib, "call", fake_call)
    monkeypatch.setattr(_lib, "require_cuda", lambda *t: None)
    monkeypatch.setattr(_lib, "stream_of", lambda t: ctypes.c_void_p(0))
    seed = lambda dev, n: (123, 0)
    monkeypatch.setattr(_rng, "philox_seed_offset", seed)
    import nmtgminor_amd.native._attn_common as ac
    import nmtgminor_amd.native._mlp_common as mc
    import nmtgminor_amd.native.fused_dropout_add_cuda as dac
    import nmtgminor_amd.native.mask_softmax_dropout_cuda as smc
    for m in (ac, mc, dac, smc):
        if hasattr(m, "philox_seed_offset"):
            monkeypatch.setattr(m, "philox_seed_offset", seed)
