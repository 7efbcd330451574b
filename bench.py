#!/usr/bin/env python3
"""Benchmark of the fused transformer-layer ops on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME|all] [--no-cpu]

A "step" is one forward+backward pass (forward only where the workload says so) of one op over
one batch of seeded synthetic input already resident in HBM. The headline line is the fused-MLP
workload (MFMA TFLOP/s); with `--workload all` (the default) the other benchmark workloads are
measured too and reported under "others", each with its own roofline and CPU baseline.

Timing: W warm-up steps, then exactly K steps replayed from a HIP graph of one step, bracketed by
device synchronisation; per-kernel durations come from HIP events the library records around
each launch (nmtg_trace_begin/end) in a separate eager pass, so they can be compared with a
rocprofv3 kernel trace of the same command. The CPU baseline is the CPU oracle (oracle/, a
restatement of the reference's PyTorch fallback) on the host cores, on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0       # MI355X dense bf16 / fp16 MFMA, published


def _sync():
    torch.cuda.synchronize()


class Workload:
    name = ""
    bound = "hbm"               # or "mfma"
    dtype = "f32"
    description = ""
    data = "synthetic"

    def setup(self, dev):
        raise NotImplementedError

    def step(self):
        raise NotImplementedError

    def work_per_step(self):    # bytes (hbm) or flops (mfma), algorithmic
        raise NotImplementedError

    def kernel_work(self):      # {kernel-name prefix: algorithmic work of ONE launch group per step}
        return {}

    def cpu_baseline(self):     # -> dict(value, unit, cores, kind, sample)
        return None

    @property
    def unit(self):
        return "GB/s" if self.bound == "hbm" else "TFLOP/s"

    @property
    def peak(self):
        return HBM_PEAK_GBS if self.bound == "hbm" else MFMA_PEAK_TFLOPS

    def rate(self, work, seconds):
        return work / seconds / (1e9 if self.bound == "hbm" else 1e12)


def _time_cpu(fn, reps=3):
    fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


class LayerNormWL(Workload):
    name = "layer_norm"
    bound = "hbm"
    dtype = "f32"
    description = "LayerNorm fwd+bwd fp32 [4096 x 512], eps 1e-5"

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.native import fast_layer_norm_cuda as ln
        self.ln = ln
        self.cpu = inputs.layer_norm_inputs()
        d = self.cpu
        self.x, self.g, self.b, self.dy = (d[k].to(dev) for k in ("x", "gamma", "beta", "dy"))
        self.rows, self.h = self.x.shape

    def step(self):
        z, mu, rs = self.ln.ln_fwd(self.x, self.g, self.b, 1e-5)
        return self.ln.ln_bwd(self.dy, self.x, mu, rs, self.g, None, False)

    def _bytes(self):
        t = self.rows * self.h * 4
        fwd = 2 * t + 2 * self.h * 4 + 2 * self.rows * 4
        bwd = 3 * t + 2 * self.rows * 4 + 3 * self.h * 4
        return fwd, bwd

    def work_per_step(self):
        return sum(self._bytes())

    def kernel_work(self):
        fwd, bwd = self._bytes()
        return {"ln_fwd": fwd, "ln_bwd": bwd}

    def cpu_baseline(self):
        from oracle import layer_norm as o
        d = self.cpu

        def run():
            z, mu, rs = o.ln_fwd(d["x"], d["gamma"], d["beta"], d["eps"])
            o.ln_bwd(d["dy"], d["x"], mu, rs, d["gamma"])
        t = _time_cpu(run, 5)
        return dict(value=self.work_per_step() / t / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                    sample="full workload (4096 x 512 fp32 fwd+bwd), median of 5")


class LayerNormLargeWL(LayerNormWL):
    """The streaming rate of the LayerNorm kernels on tensors beyond the 256 MB last-level cache: 64 times the rows
    of the largest shape the reference's own timing script uses (512 * 32 rows of 1024, onmt/modules/test_layer_norm.py:243-255),
    in bf16 with bf16 weights."""
    name = "layer_norm_large"
    dtype = "bf16"
    description = "LayerNorm fwd+bwd bf16 [65536 x 1024], eps 1e-5 (134 MB per tensor: beyond the last-level cache)"

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.native import fast_layer_norm_cuda as ln
        self.ln = ln
        self.cpu = inputs.layer_norm_inputs(65536, 1024, torch.bfloat16, seed=1011)
        d = self.cpu
        self.x, self.g, self.b, self.dy = (d[k].to(dev) for k in ("x", "gamma", "beta", "dy"))
        self.rows, self.h = self.x.shape

    def _bytes(self):
        t = self.rows * self.h * 2
        fwd = 2 * t + 2 * self.h * 2 + 2 * self.rows * 4
        bwd = 3 * t + 2 * self.rows * 4 + 3 * self.h * 2
        return fwd, bwd

    def cpu_baseline(self):
        from oracle import layer_norm as o
        d = self.cpu
        rows = 8192                                   # a bounded sample: one eighth of the rows

        def run():
            z, mu, rs = o.ln_fwd(d["x"][:rows], d["gamma"], d["beta"], d["eps"])
            o.ln_bwd(d["dy"][:rows], d["x"][:rows], mu, rs, d["gamma"])
        t = _time_cpu(run, 3)
        return dict(value=self.work_per_step() * rows / self.rows / t / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                    sample="the first 8192 of 65536 rows, fwd+bwd in fp32 on the bf16 values, median of 3")


class MlpWL(Workload):
    name = "mlp"
    bound = "mfma"
    dtype = "f16"
    description = "fused MLP fwd+bwd fp16: x [8192 x 512], 512->2048->512, gelu, dropout 0.1 (explicit mask)"

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.native import fused_mlp_gelu as m
        self.m = m
        self.cpu = inputs.mlp_inputs()
        d = self.cpu
        self.ins = [d[k].to(dev) for k in ("x", "w1", "w2", "b1", "b2")]
        self.ins[0].requires_grad_()
        self.mask = d["mask"].to(dev)
        self.dy = d["dy"].to(dev)

    def step(self):
        out = self.m.forward(0.1, self.ins, self.mask)
        return self.m.backward(0.1, self.dy, out, self.ins)

    def work_per_step(self):
        return 6 * 2.0 * 8192 * 512 * 2048

    def kernel_work(self):
        return {"gemm_": self.work_per_step()}

    def cpu_baseline(self):
        from oracle import mlp as o
        d = self.cpu
        ws, bs = [d["w1"].float(), d["w2"].float()], [d["b1"].float(), d["b2"].float()]
        x, dy = d["x"].float(), d["dy"].float()

        def run():
            y, pre, post = o.mlp_fwd(x, ws, bs, "gelu", 0.1, [d["mask"]])
            o.mlp_bwd(dy, x, ws, pre, post, "gelu", 0.1, [d["mask"]])
        t = _time_cpu(run, 3)
        return dict(value=self.work_per_step() / t / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                    sample="full workload in fp32 on the fp16-rounded values, median of 3")


class XentropyWL(Workload):
    name = "xentropy"
    bound = "hbm"
    dtype = "bf16"
    description = ("label-smoothed cross-entropy fwd+bwd: bf16 logits [16384 x 250054], eps 0.1, "
                   "10% padding (idx 1), fp32 accumulation")
    data = "synthetic (logits drawn on the GPU by torch's Philox generator, seed 1005; targets from the seeded CPU generator)"
    rows, vocab = 16384, 250054

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.native import xentropy_cuda as xe
        self.xe = xe
        d = inputs.xentropy_inputs(self.rows, self.vocab, with_logits=False)
        self.labels_cpu = d["labels"]
        self.labels = d["labels"].to(dev)
        self.grad = d["grad_loss"].to(dev)
        g = torch.Generator(device=dev)
        g.manual_seed(1005)
        self.logits = torch.empty(self.rows, self.vocab, dtype=torch.bfloat16, device=dev)
        chunk = 1024
        for r in range(0, self.rows, chunk):
            self.logits[r:r + chunk] = (2.0 * torch.randn(chunk, self.vocab, generator=g, device=dev)).to(torch.bfloat16)
        self.grad_logits = None

    def step(self):
        losses, lse = self.xe.forward(self.logits, self.labels, 0.1, True, padding_idx=1)
        g = self.xe.backward(self.grad, self.logits, lse, self.labels, 0.1, padding_idx=1)
        return losses, g

    def _tensor_bytes(self):
        return self.rows * self.vocab * 2

    def work_per_step(self):
        return 3 * self._tensor_bytes()

    def kernel_work(self):
        return {"xentropy_fwd": self._tensor_bytes(), "xentropy_bwd": 2 * self._tensor_bytes()}

    def cpu_baseline(self):
        from oracle import xentropy as o
        n = 256
        x = self.logits[:n].float().cpu()
        y = self.labels_cpu[:n]
        gl = torch.ones(n)

        def run():
            loss, lse = o.xentropy_fwd(x, y, 0.1, 1)
            o.xentropy_bwd(gl, x, lse, y, 0.1, 1)
        t = _time_cpu(run, 3)
        return dict(value=3 * n * self.vocab * 2 / t / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                    sample=f"first {n} of {self.rows} rows, fp32 on the bf16-rounded logits, algorithmic bf16 bytes / time, median of 3")


class SelfAttnWL(Workload):
    name = "self_attn"
    bound = "mfma"
    dtype = "bf16"
    description = ("encoder self-attention fwd+bwd bf16: T=512, B=32, E=1024, 16 heads, key-padding lengths U[256,512], "
                   "softmax dropout 0.1 (explicit mask)")
    T, B, E, H = 512, 32, 1024, 16

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.native import self_multihead_attn_blaslt as m
        self.m = m
        d = inputs.self_attn_inputs(self.T, self.B, self.E, self.H)
        self.cpu = d
        g = lambda k: d[k].to(dev)
        self.x, self.w_in, self.w_out, self.b_in, self.b_out = g("x"), g("w_in"), g("w_out"), g("b_in"), g("b_out")
        self.pad, self.dm, self.dout = g("pad_mask"), g("dropout_mask"), g("dout")

    def step(self):
        lin, scores, dropped, dmask, ctx, out = self.m.forward(False, True, self.H, self.x, self.w_in, self.w_out, self.b_in,
                                                               self.b_out, self.pad, 0.1, dropout_mask=self.dm)
        return self.m.backward(False, self.H, self.dout, ctx, dropped, scores, lin, self.x, self.w_in, self.w_out, dmask, 0.1)

    def _flops_fwd(self):
        t, b, e, h = self.T, self.B, self.E, self.H
        tok = t * b
        return 2.0 * tok * e * 3 * e + 2 * (2.0 * b * h * t * t * (e // h)) + 2.0 * tok * e * e

    def work_per_step(self):
        return 3 * self._flops_fwd()

    def kernel_work(self):
        return {"gemm_": self.work_per_step()}

    def cpu_baseline(self):
        from oracle import attention as o
        d = self.cpu
        nb = 2                                                   # batch columns are independent
        sl = lambda z: z[:, :nb].float()
        x, dout = sl(d["x"]), sl(d["dout"])
        w_in, w_out, b_in, b_out = (d[k].float() for k in ("w_in", "w_out", "b_in", "b_out"))
        pad, dm = d["pad_mask"][:nb], d["dropout_mask"][:nb * self.H]

        def run():
            f = o.self_attn_fwd(x, w_in, w_out, b_in, b_out, self.H, pad, None, 0.1, dm)
            o.self_attn_bwd(dout, x, w_in, w_out, self.H, f, 0.1, dm)
        t = _time_cpu(run, 3)
        return dict(value=self.work_per_step() * nb / self.B / t / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(),
                    kind="port", sample=f"{nb} of {self.B} batch columns (independent), fp32 on the bf16-rounded values, median of 3")


class _PlainCtx:
    """What an autograd function's forward / backward need of their ctx, for a step that calls the two directly."""

    def save_for_backward(self, *tensors):
        self.saved_tensors = tensors


class SelfAttnNoCoverageWL(SelfAttnWL):
    name = "self_attn_no_coverage"
    description = ("the self_attn workload as self_attn_func runs it in training with return_coverage=False: projections as "
                   "GEMMs, attention core as tiled kernels over the padded batch, no [B*H, T, T] tensor (same inputs, mask, "
                   "explicit dropout mask and FLOP count as self_attn)")

    def setup(self, dev):
        super().setup(dev)
        from nmtgminor_amd.modules.flash_core import SelfAttnFlashFunc
        self.fn = SelfAttnFlashFunc
        self.w_in.requires_grad_()

    def step(self):
        with torch.no_grad():
            c = _PlainCtx()
            self.fn.forward(c, False, self.H, self.x, self.w_in, self.w_out, self.b_in, self.b_out, self.pad, 0.1, self.dm)
            return self.fn.backward(c, self.dout)

    def kernel_work(self):
        t, b, e, h = self.T, self.B, self.E, self.H
        core = 2 * (2.0 * b * h * t * t * (e // h))
        return {"gemm_": 3 * (self._flops_fwd() - core), "flash_attn_bwd": 2 * core}


class SelfAttnTimeMaskWL(SelfAttnNoCoverageWL):
    """Not part of the default run (`--workload self_attn_time_mask`): the decoder's self-attention in training."""
    name = "self_attn_time_mask"
    description = ("decoder self-attention in training, return_coverage=False: the self_attn shapes (T=512, B=32, E=1024, 16 heads) "
                   "under a causal time mask [T, T] instead of the key-padding mask, explicit dropout mask; tiled kernels that read "
                   "the mask as packed words; FLOPs counted dense, as the reference computes them under a mask")

    def setup(self, dev):
        super().setup(dev)
        self.tmask = torch.triu(torch.ones(self.T, self.T, dtype=torch.bool), 1).to(dev)

    def step(self):
        with torch.no_grad():
            c = _PlainCtx()
            self.fn.forward(c, True, self.H, self.x, self.w_in, self.w_out, self.b_in, self.b_out, self.tmask, 0.1, self.dm)
            return self.fn.backward(c, self.dout)

    def cpu_baseline(self):
        from oracle import attention as o
        d = self.cpu
        nb = 2
        sl = lambda z: z[:, :nb].float()
        x, dout = sl(d["x"]), sl(d["dout"])
        w_in, w_out, b_in, b_out = (d[k].float() for k in ("w_in", "w_out", "b_in", "b_out"))
        tm, dm = torch.triu(torch.ones(self.T, self.T, dtype=torch.bool), 1), d["dropout_mask"][:nb * self.H]

        def run():
            f = o.self_attn_fwd(x, w_in, w_out, b_in, b_out, self.H, None, tm, 0.1, dm)
            o.self_attn_bwd(dout, x, w_in, w_out, self.H, f, 0.1, dm)
        t = _time_cpu(run, 3)
        return dict(value=self.work_per_step() * nb / self.B / t / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(),
                    kind="port", sample=f"{nb} of {self.B} batch columns (independent), fp32 on the bf16-rounded values, median of 3")


class FlashAttnWL(Workload):
    name = "flash_attn"
    bound = "mfma"
    dtype = "bf16"
    description = ("attention core over packed sequences fwd+bwd bf16 (no [heads, T, T] tensor): 32 sequences of lengths "
                   "U[256,512] packed as [tokens, 3, 16 heads, 64], softmax dropout 0.1 drawn on the device")
    B, H, D, P = 32, 16, 64, 0.1

    def setup(self, dev):
        from nmtgminor_amd.native import flash_attn_cuda as m
        self.m = m
        g = torch.Generator().manual_seed(5)
        self.lens = torch.randint(256, 513, (self.B,), generator=g).tolist()
        cu = torch.zeros(self.B + 1, dtype=torch.int32)
        cu[1:] = torch.cumsum(torch.tensor(self.lens), 0)
        total = int(cu[-1])
        self.cpu = dict(qkv=torch.randn(total, 3, self.H, self.D, generator=g).to(torch.bfloat16),
                        dout=torch.randn(total, self.H, self.D, generator=g).to(torch.bfloat16), cu=cu)
        self.qkv, self.dout, self.cu = self.cpu["qkv"].to(dev), self.cpu["dout"].to(dev), cu.to(dev)
        self.out = torch.empty_like(self.dout)
        self.dqkv = torch.empty_like(self.qkv)
        self.max_len = max(self.lens)
        self.scale = self.D ** -0.5

    def step(self):
        q, k, v = self.qkv[:, 0], self.qkv[:, 1], self.qkv[:, 2]
        lse, = self.m.fwd(q, k, v, self.out, self.cu, self.cu, self.max_len, self.max_len, self.P, self.scale, False, False,
                          False, rng=(20250101, 0))        # a fixed Philox state: the step is captured into a graph
        return self.m.bwd(self.dout, q, k, v, self.out, lse, self.dqkv[:, 0], self.dqkv[:, 1], self.dqkv[:, 2], self.cu, self.cu,
                          self.max_len, self.max_len, self.P, self.scale, False, False, rng=self.m.last_rng)   # with the forward's keep bits

    def _flops_fwd(self):
        return sum(2 * 2.0 * self.H * n * n * self.D for n in self.lens)        # Q K^T and P V per sequence and head

    def work_per_step(self):
        return 3 * self._flops_fwd()                                            # backward: dP, dV, dQ, dK

    def kernel_work(self):
        return {"flash_attn_fwd": self._flops_fwd(), "flash_attn_bwd": 2 * self._flops_fwd()}

    def cpu_baseline(self):
        from oracle import flash_attention as o
        nb = 2
        cu = self.cpu["cu"][:nb + 1]
        n = int(cu[-1])
        qkv, dout = self.cpu["qkv"][:n].float(), self.cpu["dout"][:n].float()
        keep = (torch.rand(nb, self.H, self.max_len, self.max_len, generator=torch.Generator().manual_seed(6)) >= self.P).to(torch.uint8)

        def run():
            o.flash_attn_bwd(dout, qkv[:, 0], qkv[:, 1], qkv[:, 2], cu, cu, self.max_len, None, False, self.P, keep, torch.float32)
        t = _time_cpu(run, 3)
        work = 3 * sum(2 * 2.0 * self.H * x * x * self.D for x in self.lens[:nb])
        return dict(value=work / t / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                    sample=f"{nb} of {self.B} sequences (independent), fp32 on the bf16-rounded values, forward + autograd backward, median of 3")


class RelSelfAttnWL(Workload):
    name = "rel_self_attn"
    bound = "mfma"
    dtype = "bf16"
    description = ("self-attention with relative positions fwd+bwd bf16 (speech-encoder form): T=512, B=32, E=1024, 16 heads, "
                   "R=512 positions shared over the batch, key-padding lengths U[256,512], softmax dropout 0.1 (explicit mask)")
    T, B, E, H = 512, 32, 1024, 16
    NAMES = ("x", "pos", "w_in", "w_out", "w_pos", "b_in", "b_out", "b_pos", "r_w_bias", "r_r_bias")

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.modules.relative_self_attention_func import relative_self_attn_func
        self.fn = relative_self_attn_func
        d = inputs.rel_self_attn_inputs(self.T, self.B, self.E, self.H, torch.bfloat16, p=0.1, seed=1006)
        self.cpu = d
        self.t = {k: d[k].to(dev).requires_grad_(k != "pos") for k in self.NAMES}
        self.pad, self.dm, self.dout = d["pad_mask"].to(dev), d["dropout_mask"].to(dev), d["dout"].to(dev)

    def step(self):
        t = self.t
        for v in t.values():
            v.grad = None
        out = self.fn(t["x"], t["pos"], False, True, self.H, t["w_in"], t["w_out"], t["w_pos"], t["b_in"], t["b_out"],
                      t["b_pos"], t["r_w_bias"], t["r_r_bias"], self.pad, 0.1, False, None, False, False, False, False, self.dm)
        out.backward(self.dout)
        return t["x"].grad

    def _flops_fwd(self):
        t, b, e, h = self.T, self.B, self.E, self.H
        tok = t * b
        # in-projection, position projection (per batch column, as the reference lays it out), AC, BD, P V, out-projection
        return 2.0 * tok * e * 3 * e + 2.0 * tok * e * e + 3 * (2.0 * b * h * t * t * (e // h)) + 2.0 * tok * e * e

    def work_per_step(self):
        # backward: two products per forward product, except the position projection (weight gradient only)
        return 3 * self._flops_fwd() - 2.0 * self.T * self.B * self.E * self.E

    def kernel_work(self):
        return {"gemm_": self.work_per_step()}

    def cpu_baseline(self):
        from oracle import relative_attention as o
        d = self.cpu
        nb = 2                                                   # batch columns are independent
        a = {k: d[k].float() for k in self.NAMES}
        a["x"] = a["x"][:, :nb]
        dout, pad, dm = d["dout"][:, :nb].float(), d["pad_mask"][:nb], d["dropout_mask"][:nb * self.H]

        def run():
            f = o.rel_self_attn_fwd(*(a[k] for k in self.NAMES), self.H, pad, None, 0.1, dm)
            o.rel_self_attn_bwd(dout, a["x"], a["pos"], a["w_in"], a["w_out"], a["w_pos"], self.H, f, 0.1, dm)
        t = _time_cpu(run, 3)
        return dict(value=self.work_per_step() * nb / self.B / t / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(),
                    kind="port", sample=f"{nb} of {self.B} batch columns (independent), fp32 on the bf16-rounded values, median of 3")


class EncdecAttnWL(Workload):
    name = "encdec_attn"
    bound = "mfma"
    dtype = "bf16"
    description = ("decoder layer attention fwd bf16: cross-attention Tq=128 over Tk=1500 (B=16, E=1024, 16 heads, key lengths "
                   "U[750,1500]) + causal self-attention T=128; eval (no dropout)")
    TQ, TK, B, E, H = 128, 1500, 16, 1024, 16

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.native import encdec_multihead_attn_bias_blaslt as m, self_multihead_attn_blaslt as sm
        self.m, self.sm = m, sm
        d = inputs.encdec_attn_inputs(self.TQ, self.TK, self.B, self.E, self.H)
        s = inputs.self_attn_inputs(self.TQ, self.B, self.E, self.H, p=0.0, seed=1004, causal=True)
        self.cpu, self.cpu_self = d, s
        self.a = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in d.items()}
        self.s = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in s.items()}

    def step(self):
        s, a = self.s, self.a
        with torch.no_grad():            # inference, as the reference's translator runs its decoder
            r1 = self.sm.forward(True, False, self.H, s["x"], s["w_in"], s["w_out"], s["b_in"], s["b_out"], s["time_mask"], 0.0)
            r2 = self.m.forward(False, self.H, a["x_q"], a["x_kv"], a["w_q"], a["w_kv"], a["w_out"], a["b_q"], a["b_kv"],
                                a["b_out"], a["pad_mask"], 0.0)
        return r1[-1], r2[-1]

    def work_per_step(self):
        tq, tk, b, e, h = self.TQ, self.TK, self.B, self.E, self.H
        d = e // h
        cross = 2.0 * tq * b * e * e + 2.0 * tk * b * e * 2 * e + 2 * (2.0 * b * h * tq * tk * d) + 2.0 * tq * b * e * e
        self_ = 2.0 * tq * b * e * 3 * e + 2 * (2.0 * b * h * tq * tq * d) + 2.0 * tq * b * e * e
        return cross + self_

    def kernel_work(self):
        return {"gemm_": self.work_per_step()}

    def cpu_baseline(self):
        from oracle import attention as o
        d, s = self.cpu, self.cpu_self
        f = lambda z: z.float() if z is not None and z.is_floating_point() else z

        def run():
            o.self_attn_fwd(f(s["x"]), f(s["w_in"]), f(s["w_out"]), f(s["b_in"]), f(s["b_out"]), self.H, None, s["time_mask"])
            o.encdec_attn_fwd(f(d["x_q"]), f(d["x_kv"]), f(d["w_q"]), f(d["w_kv"]), f(d["w_out"]), f(d["b_q"]), f(d["b_kv"]),
                              f(d["b_out"]), self.H, d["pad_mask"])
        t = _time_cpu(run, 3)
        return dict(value=self.work_per_step() / t / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                    sample="full workload in fp32 on the bf16-rounded values, median of 3")



class DecodeStepWL(Workload):
    name = "decode_step"
    bound = "hbm"
    dtype = "bf16"
    description = ("one incremental decoding step of the decoder's attention, bf16: cross-attention of 1 new position over "
                   "1500 cached encoder keys / values (B=32 hypotheses, E=1024, 16 heads, key-padding lengths U[750,1500]: bytes counted over the live keys) + "
                   "self-attention of the new position over 127 cached positions (the step starts from a cache tensor without room to grow, so it copies the cache once, as the reference's concatenation does)")
    TK, TPREV, B, E, H = 1500, 127, 32, 1024, 16

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.modules import incremental as inc
        self.inc = inc
        d = inputs.encdec_attn_inputs(1, self.TK, self.B, self.E, self.H, seed=1010)
        s = inputs.self_attn_inputs(self.TPREV + 1, self.B, self.E, self.H, p=0.0, seed=1011)
        self.cpu, self.cpu_self = d, s
        self.a = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in d.items()}
        self.s = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in s.items()}
        self.cross_cache, self_cache = {}, {}
        a, sa = self.a, self.s
        inc.encdec_attn_step(self.H, a["x_q"], a["x_kv"], a["w_q"], a["w_kv"], a["w_out"], a["b_q"], a["b_kv"], a["b_out"],
                             a["pad_mask"], self.cross_cache)                       # fills c_k / c_v: not part of a step
        inc.self_attn_step(self.H, sa["x"][:self.TPREV], sa["w_in"], sa["w_out"], sa["b_in"], sa["b_out"], None, self_cache, False)
        self.prev_k, self.prev_v = self_cache["k"], self_cache["v"]
        # the cache rows a step has to read: the live keys of every sentence (the kernel does not read a sentence's padding)
        self.live_keys = int((~d["pad_mask"].bool()).sum())

    def step(self):
        a, sa = self.a, self.s
        cache = {"k": self.prev_k, "v": self.prev_v}                                  # every step appends to the same 127 positions
        r1 = self.inc.self_attn_step(self.H, sa["x"][self.TPREV:], sa["w_in"], sa["w_out"], sa["b_in"], sa["b_out"], None, cache,
                                     False)
        r2 = self.inc.encdec_attn_step(self.H, a["x_q"], None, a["w_q"], None, a["w_out"], a["b_q"], None, a["b_out"],
                                       a["pad_mask"], self.cross_cache)
        return r1[0], r2[0]

    def _bytes(self):
        tk, tp, b, e, h = self.TK, self.TPREV, self.B, self.E, self.H
        cross = 2 * self.live_keys * e * 2 + 2 * e * e * 2 + b * h * tk * 2 + 4 * b * e * 2  # live K, V rows; W_q, W_out; probabilities; rows
        self_ = 2 * (tp + tp + 1) * b * e * 2 + 4 * e * e * 2 + b * h * (tp + 1) * 2 + 5 * b * e * 2   # cache read + rewritten
        return cross + self_

    def work_per_step(self):
        return self._bytes()

    def kernel_work(self):
        tk, tp, b, e, h = self.TK, self.TPREV, self.B, self.E, self.H
        # the two launches of the cache-streaming kernel: keys and values read once, probabilities written, a row in and out
        return {"attn_decode": 2 * (self.live_keys + (tp + 1) * b) * e * 2 + b * h * (tk + tp + 1) * 2 + 4 * b * e * 2}

    def cpu_baseline(self):
        from oracle import attention as o
        d, s = self.cpu, self.cpu_self
        f = lambda z: z.float() if z is not None and z.is_floating_point() else z
        kv = (f(d["x_kv"]).view(-1, self.E) @ f(d["w_kv"]).t()).view(self.TK, self.B, 2 * self.E)   # the cached projection

        def run():
            # the step's arithmetic: the new position's row of both attentions, keys / values already projected
            o.self_attn_fwd(f(s["x"]), f(s["w_in"]), f(s["w_out"]), f(s["b_in"]), f(s["b_out"]), self.H, None, None)
            q = f(d["x_q"]).view(-1, self.E) @ f(d["w_q"]).t()
            dd = self.E // self.H
            k4 = kv.view(self.TK, self.B * self.H, 2, dd)
            sc = torch.einsum("bd,tbd->bt", q.view(self.B * self.H, dd), k4[:, :, 0]) * dd ** -0.5
            pr = torch.softmax(sc.masked_fill(d["pad_mask"].repeat_interleave(self.H, 0), float("-inf")), -1)
            ctx = torch.einsum("bt,tbd->bd", pr, k4[:, :, 1]).reshape(self.B, self.E)
            return ctx @ f(d["w_out"]).t()
        t = _time_cpu(run, 3)
        return dict(value=self._bytes() / t / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                    sample="full step in fp32 on the bf16-rounded values (self-attention recomputed over its 128 positions), median of 3")


class SoftmaxDropoutWL(Workload):
    name = "softmax_dropout"
    bound = "hbm"
    dtype = "bf16"
    description = ("masked softmax + dropout as its own op, fwd + recomputing bwd, bf16 scores [512 x 512 x 512] "
                   "(32 sentences x 16 heads), key-padding mask, dropout 0.1 (explicit mask)")
    HEADS, BATCH, T = 16, 32, 512

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.native import mask_softmax_dropout_cuda as sm
        self.sm = sm
        g = torch.Generator().manual_seed(1003)
        self.heads, b, t = self.HEADS, self.BATCH, self.T
        bh = b * self.heads
        self.cpu_scores = (torch.randn(bh, t, t, generator=g) * 3).to(torch.bfloat16)
        self.cpu_pad, _ = inputs.lengths_mask(b, t, t // 2, t, g)
        self.cpu_dm = inputs.bernoulli_mask((bh, t, t), 0.9, g)
        self.cpu_go = torch.randn(bh, t, t, generator=g).to(torch.bfloat16)
        self.s, self.pad, self.dm, self.go = (v.to(dev) for v in (self.cpu_scores, self.cpu_pad, self.cpu_dm, self.cpu_go))
        self.n = self.s.numel()

    def step(self):
        _, _, dropped = self.sm.forward(True, self.heads, self.s, 0.1, pad_mask=self.pad, dropout_mask=self.dm,
                                        want_softmax=False)
        ds = self.sm.backward_recompute(self.heads, self.go, None, self.s, self.dm, 0.1, pad_mask=self.pad)
        return dropped, ds

    def _bytes(self):
        # fwd: scores read, dropped probabilities written, dropout mask read; bwd: gradient and scores read, mask read,
        # gradient of the scores written (the key-padding mask is 16 KB)
        return 5 * self.n, 7 * self.n

    def work_per_step(self):
        return sum(self._bytes())

    def kernel_work(self):
        fwd, bwd = self._bytes()
        return {"softmax_dropout_fwd": fwd, "softmax_dropout_bwd": bwd}

    def cpu_baseline(self):
        from oracle import softmax_dropout as o
        rows = self.heads                           # the 16 heads of the first sentence, of 512 (sentence, head) slices
        s, dm, go = self.cpu_scores[:rows], self.cpu_dm[:rows], self.cpu_go[:rows]
        pad = self.cpu_pad[:1]

        def run():
            masked = o.masked_scores(s.float(), pad_mask=pad, heads=rows)
            sm_, _ = o.softmax_dropout_fwd(masked, dm, 0.1)
            o.softmax_dropout_bwd(go, sm_, dm, 0.1)
        t = _time_cpu(run, 3)
        return dict(value=self.work_per_step() * rows / self.s.shape[0] / t / 1e9, unit="GB/s", cores=torch.get_num_threads(),
                    kind="port", sample="the first sentence (16 of the 512 [512 x 512] slices), fwd+bwd, median of 3")


class DropoutAddWL(Workload):
    name = "dropout_add"
    bound = "hbm"
    dtype = "bf16"
    description = "dropout + residual add fwd+bwd bf16 [512 x 32 x 1024], dropout 0.1 (explicit mask), in place"
    SHAPE = (512, 32, 1024)

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.native import fused_dropout_add_cuda as da
        self.da = da
        g = torch.Generator().manual_seed(1006)
        shape = self.SHAPE
        self.cpu_x = torch.randn(shape, generator=g).to(torch.bfloat16)
        self.cpu_r = torch.randn(shape, generator=g).to(torch.bfloat16)
        self.cpu_m = inputs.bernoulli_mask(shape, 0.9, g)
        self.cpu_g = torch.randn(shape, generator=g).to(torch.bfloat16)
        self.x0, self.r, self.m, self.g = (v.to(dev) for v in (self.cpu_x, self.cpu_r, self.cpu_m, self.cpu_g))
        self.x = self.x0.clone()
        self.n = self.x.numel()

    def step(self):
        # in place, as the reference: x <- dropout(x) + residual. The buffer is reused from step to step; its values
        # stay finite (a random walk of unit steps over the run) and do not influence the time.
        mask, out = self.da.forward(True, self.x, self.r, 0.1, self.m)
        dx = self.da.backward(self.g, mask, 0.1)
        return out, dx

    def _bytes(self):
        return 7 * self.n, 5 * self.n     # fwd: x, residual read + x written (2 B each) + mask; bwd: g read, dx written + mask

    def work_per_step(self):
        return sum(self._bytes())

    def kernel_work(self):
        fwd, bwd = self._bytes()
        return {"dropout_add_fwd": fwd, "dropout_add_bwd": bwd}

    def cpu_baseline(self):
        from oracle import dropout_add as o
        x, r, m, g = self.cpu_x, self.cpu_r, self.cpu_m, self.cpu_g

        def run():
            o.dropout_add_fwd(x, r, m, 0.1)
            o.dropout_add_bwd(g, m, 0.1)
        t = _time_cpu(run, 3)
        return dict(value=self.work_per_step() / t / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                    sample="full workload ([512 x 32 x 1024] bf16 fwd+bwd), median of 3")


class FusedAdamWL(Workload):
    name = "fused_adam"
    bound = "hbm"
    dtype = "f32"
    description = ("AdamW update of a transformer-base parameter list in fp32: 6 + 6 layers of E=512 / inner 2048 weights and "
                   "biases plus a 32000 x 512 embedding, 193 tensors, 60.5 M elements, one multi-tensor pass")
    E, INNER, VOCAB, LAYERS = 512, 2048, 32000, 12

    def shapes(self):
        e, f = self.E, self.INNER
        per_layer = [(3 * e, e), (3 * e,), (e, e), (e,), (f, e), (f,), (e, f), (e,), (e,), (e,), (e,), (e,)]
        # decoder layers carry a cross-attention block as well
        cross = [(e, e), (e,), (2 * e, e), (2 * e,), (e, e), (e,), (e,), (e,)]
        out = [(self.VOCAB, e)]
        for i in range(self.LAYERS):
            out += per_layer + (cross if i >= self.LAYERS // 2 else [])
        return out

    def setup(self, dev):
        from nmtgminor_amd.native import fused_optim
        self.op = fused_optim.multi_tensor_adam
        g = torch.Generator(device=dev).manual_seed(1007)
        mk = lambda s, scale: scale * torch.randn(s, generator=g, device=dev)
        shapes = self.shapes()
        self.lists = [[mk(s, 1e-2) for s in shapes], [mk(s, 0.1) for s in shapes], [mk(s, 1e-3) for s in shapes],
                      [mk(s, 1e-3).abs() for s in shapes]]
        self.n = sum(t.numel() for t in self.lists[0])
        self.step_no = 0

    def step(self):
        self.step_no += 1
        self.op(65536, None, self.lists, 1e-4, 0.9, 0.98, 1e-8, self.step_no, 1, 1, 0.01)
        return self.lists[1][0]

    def work_per_step(self):
        return 7 * 4 * self.n                                # g, p, m, v read; p, m, v written

    def kernel_work(self):
        return {"multi_tensor_adam": self.work_per_step()}

    def cpu_baseline(self):
        from oracle import fused_optim as o
        k = 24                                               # the first tensors: the embedding and two layers
        lists = [[t.detach().cpu() for t in lst[:k]] for lst in self.lists]
        n = sum(t.numel() for t in lists[0])

        def run():
            for g, p, m, v in zip(*lists):
                o.adam_step(g, p, m, v, 1e-4, 0.9, 0.98, 1e-8, 3, 1, True, 0.01)
        t = _time_cpu(run, 3)
        return dict(value=7 * 4 * n / t / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                    sample=f"the first {k} of {len(self.lists[0])} tensors ({n} elements), fp32, median of 3")


class GeneratorLossWL(Workload):
    name = "generator_loss"
    bound = "mfma"
    dtype = "bf16"
    description = ("output projection + label-smoothed cross-entropy fwd+bwd, the bf16 logits kept once in HBM (8.2 GB) and "
                   "turned into their gradient in place: bf16 states [16384 x 1024], vocabulary 250054, eps 0.1, 10% padding (idx 1)")
    ROWS, MODEL, VOCAB, CHUNK = 16384, 1024, 250054, 4096

    def setup(self, dev):
        from nmtgminor_amd import synthetic as inputs
        from nmtgminor_amd.modules.generator_loss import LinearSoftmaxCrossEntropy
        self.fn = LinearSoftmaxCrossEntropy
        n, e, v = self.ROWS, self.MODEL, self.VOCAB
        d = inputs.xentropy_inputs(n, v, with_logits=False)
        self.labels_cpu = d["labels"]
        self.labels, self.grad = d["labels"].to(dev), d["grad_loss"].to(dev)
        g = torch.Generator(device=dev)
        g.manual_seed(1006)
        self.h = torch.randn(n, e, generator=g, device=dev).to(torch.bfloat16).requires_grad_()
        self.w = (torch.randn(v, e, generator=g, device=dev) / e ** 0.5).to(torch.bfloat16).requires_grad_()

    def step(self):
        self.h.grad = self.w.grad = None
        losses = self.fn.apply(self.h, self.w, None, self.labels, 0.1, 1, self.CHUNK)
        losses.backward(self.grad)
        return losses, self.h.grad, self.w.grad

    def work_per_step(self):
        # the projection and the two gradient contractions
        return 3 * 2.0 * self.ROWS * self.MODEL * self.VOCAB

    def kernel_work(self):
        return {"gemm_": self.work_per_step()}

    def cpu_baseline(self):
        from oracle import generator_loss as o
        n = 128
        h, w = self.h[:n].detach().float().cpu(), self.w.detach().float().cpu()
        y, gl = self.labels_cpu[:n], torch.ones(n)

        def run():
            o.generator_loss_fwd(h, w, None, y, 0.1, 1)
            o.generator_loss_bwd(gl, h, w, None, y, 0.1, 1)
        t = _time_cpu(run, 3)
        # the oracle's backward computes the projection again: 4 products of n x E x V in the timed region
        return dict(value=4 * 2.0 * n * self.MODEL * self.VOCAB / t / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(),
                    kind="port", sample=f"first {n} of {self.ROWS} rows against the full vocabulary, fp32, median of 3")


class CopyWL(Workload):
    """Plain device copy of a known size: the calibration target for the rocprofv3 FETCH_SIZE /
    WRITE_SIZE counters (not part of `--workload all`)."""
    name = "copy"
    bound = "hbm"
    dtype = "f32"
    description = "torch copy of 1 GiB fp32 (1 GiB read + 1 GiB written): counter calibration"

    def setup(self, dev):
        n = 1 << 28
        self.src = torch.ones(n, dtype=torch.float32, device=dev)
        self.dst = torch.empty_like(self.src)

    def step(self):
        self.dst.copy_(self.src)
        return self.dst

    def work_per_step(self):
        return 2 * self.src.numel() * 4


class StreamProbeWL(Workload):
    """One launch of the library's streaming probe (nmtg_stream_probe): the simplest kernel with the access mix of the
    bandwidth-bound kernels (16 bytes per lane and access, four in flight, the grid covers the buffer once). Its rate is
    the practical ceiling of this HBM for that mix, the figure the roofline fractions of the streaming workloads are read
    against. Not part of `--workload all`; `--workload streams` runs the six of them."""
    bound = "hbm"
    dtype = "f32"
    MODE, STREAMS, BYTES = 0, 2, 1 << 30

    def setup(self, dev):
        from nmtgminor_amd import _lib as L
        self.L = L
        n = self.BYTES // 4
        self.a = torch.ones(n, dtype=torch.float32, device=dev)
        self.b = torch.ones(n, dtype=torch.float32, device=dev) if self.MODE == 1 else None
        blocks = L.load().nmtg_stream_probe_blocks(L.i64(self.BYTES))
        self.out = torch.empty(blocks if self.MODE == 2 else n, dtype=torch.float32, device=dev)

    def step(self):
        L = self.L
        L.call("nmtg_stream_probe", L.ptr(self.a), L.ptr(self.b), L.ptr(self.out), L.i64(self.BYTES), L.i32(self.MODE),
               L.stream_of(self.a))
        return self.out

    def work_per_step(self):
        return self.STREAMS * self.BYTES + (self.out.numel() * 4 if self.MODE == 2 else 0)

    def kernel_work(self):
        return {"stream_probe": self.work_per_step()}


def _stream_probe(name, mode, streams, nbytes, what):
    size = f"{nbytes >> 20} MiB"
    return type("StreamProbe_" + name, (StreamProbeWL,), dict(
        name=name, MODE=mode, STREAMS=streams, BYTES=nbytes,
        description=f"streaming probe, {what}, {size} per buffer (fp32 lanes, 16 B per lane and access)"))


STREAM_PROBES = [_stream_probe(n + suffix, mode, streams, nbytes, what)
                 for suffix, nbytes in (("", 1 << 30), ("_64m", 1 << 26))
                 for n, mode, streams, what in (("stream_copy", 0, 2, "one stream read and one written"),
                                                ("stream_add", 1, 3, "two streams read and one written"),
                                                ("stream_read", 2, 1, "one stream read, one float per block written"))]


# the five benchmark configurations first, then the workloads added beside them
WORKLOADS = {w.name: w for w in (LayerNormWL, MlpWL, SelfAttnWL, EncdecAttnWL, XentropyWL, SoftmaxDropoutWL, DropoutAddWL,
                                    GeneratorLossWL, RelSelfAttnWL, FusedAdamWL, LayerNormLargeWL, FlashAttnWL, DecodeStepWL,
                                    SelfAttnNoCoverageWL)}
EXTRA_WORKLOADS = {CopyWL.name: CopyWL, SelfAttnTimeMaskWL.name: SelfAttnTimeMaskWL, **{w.name: w for w in STREAM_PROBES}}
PRIMARY = "mlp"


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _cache_flushed(w, reps=20):
    """Eager steps timed one by one with HIP events, a 512 MiB fill before each so that neither the
    L2 nor the 256 MB Infinity Cache still holds the operands (the small configurations fit there).
    -> milliseconds per step, or None if it could not be measured."""
    try:
        scratch = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        total = 0.0
        for _ in range(reps):
            scratch.fill_(1)
            e0.record()
            w.step()
            e1.record()
            e1.synchronize()
            total += e0.elapsed_time(e1)
        del scratch
        return total / reps
    except Exception as e:  # pragma: no cover - supplementary figure only
        sys.stderr.write(f"[bench] {w.name}: cache-flushed timing skipped ({e})\n")
        return None


def _measured_traffic():
    """HBM bytes per step of each workload's kernel groups, measured offline with rocprofv3 --pmc FETCH_SIZE and
    --pmc WRITE_SIZE (counters cannot be read from inside this process) and scaled by what the same counters read for
    a 1 GiB copy; profiles/hbm_traffic_counters.txt holds the commands and the per-group table. roofline.traffic is
    that figure per launch of the group (bytes per step / launches per step), like roofline.achieved's work."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get("bytes_per_step", {})
    except (OSError, ValueError):
        return {}


def measure(w, dev, steps, warmup, do_cpu, trace_steps):
    from nmtgminor_amd import _lib
    w.setup(dev)
    for _ in range(max(1, warmup)):
        w.step()
    _sync()
    # Steps are captured into a HIP graph and replayed: `unroll` steps per graph, so that the fixed cost of one graph
    # launch (some 20 us here, more than a whole LayerNorm step) is spread over several steps; K steps are timed in all.
    t0 = time.perf_counter()
    w.step()
    _sync()
    est = time.perf_counter() - t0
    unroll = 1
    if est < 1e-3:
        unroll = next((u for u in (10, 5, 4, 2) if steps % u == 0), 1)
    graph = None
    try:
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            w.step()
            _sync()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=s):
                for _ in range(unroll):
                    w.step()
        _sync()
        graph.replay()
        _sync()
    except Exception as e:  # pragma: no cover - falls back to eager launches
        sys.stderr.write(f"[bench] {w.name}: graph capture failed ({e}); timing eager launches\n")
        graph = None
    _sync()
    t0 = time.perf_counter()
    if graph is not None:
        for _ in range(steps // unroll):
            graph.replay()
    else:
        for _ in range(steps):
            w.step()
    _sync()
    wall = time.perf_counter() - t0
    per_step = wall / steps
    # per-kernel durations (HIP events around every launch, eager pass)
    _lib.trace_begin()
    for _ in range(trace_steps):
        w.step()
    _sync()
    tr = _lib.trace_end()
    kernels = []
    for name, (cnt, ms) in sorted(tr.items(), key=lambda kv: -kv[1][1]):
        kernels.append(dict(name=name, launches_per_step=cnt / trace_steps, avg_us=ms / cnt * 1e3,
                            us_per_step=ms / trace_steps * 1e3))
    roof = None
    best = None
    traffic_table = _measured_traffic().get(w.name, {})
    for prefix, work in w.kernel_work().items():
        sel = [k for k in kernels if k["name"].startswith(prefix)]
        if not sel:
            continue
        us = sum(k["us_per_step"] for k in sel)
        if best is None or us > best[0]:
            best = (us, prefix, work, sel)
    if best is not None:
        us, prefix, work, sel = best
        achieved = w.rate(work, us * 1e-6)
        launches = sum(k["launches_per_step"] for k in sel)
        roof = dict(bound=w.bound, achieved=round(achieved, 3), peak=w.peak, unit=w.unit, frac=round(achieved / w.peak, 4),
                    traffic=(round(traffic_table[prefix] / launches) if traffic_table.get(prefix) and launches else None), kernel=(prefix + "*" if prefix.endswith("_") else prefix), launches_per_step=launches,
                    avg_launch_us=round(us / launches, 3), work_per_step=work)
    res = dict(workload=w.name, description=w.description, metric="achieved HBM GB/s" if w.bound == "hbm" else "MFMA TFLOP/s",
               value=round(w.rate(w.work_per_step(), per_step), 3), unit=w.unit, ms_per_step=round(per_step * 1e3, 5),
               frac_of_peak=round(w.rate(w.work_per_step(), per_step) / w.peak, 4), dtype=w.dtype, data=w.data,
               timed=(f"hip graph replay, {unroll} steps per graph" if graph is not None else "eager launches"), roofline=roof,
               kernels=[dict(name=k["name"], launches_per_step=k["launches_per_step"], avg_us=round(k["avg_us"], 3))
                        for k in kernels])
    if w.name == "layer_norm":
        # every tensor of this configuration fits the on-chip caches: also report a cold-cache figure
        ms = _cache_flushed(w)
        if ms:
            res["cache_flushed"] = dict(ms_per_step=round(ms, 5), value=round(w.rate(w.work_per_step(), ms * 1e-3), 3),
                                        unit=w.unit, timed="eager launches, 512 MiB fill before every step")
    res["cpu_baseline"] = w.cpu_baseline() if do_cpu else None
    if res["cpu_baseline"]:
        res["cpu_baseline"]["value"] = round(res["cpu_baseline"]["value"], 4)
        res["cpu_baseline"]["cpu_model"] = _cpu_model()
    return res


RESULT_TAG = "NMTG_BENCH_RESULT "
OTHER_TAG = "NMTG_BENCH_OTHER "     # full record of a workload other than the headline one (printed before the headline line)


def _run_workloads(names, args, dev, emit):
    """Measures the named workloads one after the other in this process. emit: print each result as soon as it exists
    (tagged line on stdout), so that a parent process keeps what was measured if a later workload ends the process."""
    table = dict(WORKLOADS, **EXTRA_WORKLOADS)
    results = []
    t_start = time.perf_counter()
    for n in names:
        w = table[n]()
        steps = args.steps if w.name not in ("xentropy", "generator_loss") else max(3, min(args.steps, 10))
        # the CPU baselines are the slow part of a run: once the process has used its time allowance, the remaining
        # workloads are measured on the GPU only (cpu_baseline null), so that the whole run stays within minutes
        do_cpu = not args.no_cpu and time.perf_counter() - t_start < args.cpu_time_allowance
        try:
            results.append(measure(w, dev, steps, args.warmup, do_cpu, min(args.trace_steps, steps)))
        except Exception as e:
            if n == names[0] and not emit:
                raise                    # no headline without the first workload
            sys.stderr.write(f"[bench] workload {n} failed: {e}\n")
            results.append(dict(workload=n, error=str(e)))
        results[-1]["steps"] = steps
        if emit:
            print(RESULT_TAG + json.dumps(results[-1]), flush=True)
        del w
        torch.cuda.empty_cache()
    return results


def _in_child(names, args, limit_s):
    """Runs `bench.py --in-process --emit-results` on the named workloads as a child process and collects the results it
    printed. A workload the child did not get to (it ended early, or ran into the time limit) is reported as an error
    entry, so one workload cannot take the others' measurements with it."""
    import subprocess
    cmd = [sys.executable, os.path.abspath(__file__), "--in-process", "--emit-results", "--workload", ",".join(names),
           "--steps", str(args.steps), "--warmup", str(args.warmup), "--trace-steps", str(args.trace_steps),
           "--cpu-time-allowance", str(args.cpu_time_allowance)]
    if args.no_cpu:
        cmd.append("--no-cpu")
    out, note = "", None
    try:
        r = subprocess.run(cmd, stdout=subprocess.PIPE, text=True, timeout=limit_s)
        out = r.stdout
        if r.returncode != 0:
            note = f"the measuring process ended with status {r.returncode}"
    except subprocess.TimeoutExpired as e:
        out = e.stdout if isinstance(e.stdout, str) else (e.stdout or b"").decode(errors="replace")
        note = f"the measuring process was stopped after {limit_s} s"
    got = {}
    for line in out.splitlines():
        if line.startswith(RESULT_TAG):
            try:
                r = json.loads(line[len(RESULT_TAG):])
                got[r["workload"]] = r
            except (ValueError, KeyError):
                pass
    return [got.get(n, dict(workload=n, error=note or "no result was reported")) for n in names]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", help="one or more (comma-separated) of %s, or all; beside them: copy (counter calibration) and streams (the six "
                    "streaming probes %s)" % (", ".join(WORKLOADS), ", ".join(w.name for w in STREAM_PROBES)))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--trace-steps", type=int, default=10)
    ap.add_argument("--cpu-time-allowance", type=float, default=240.0,
                    help="seconds a measuring process may have run when it starts a workload's CPU baseline; later "
                         "workloads are measured without one")
    ap.add_argument("--in-process", action="store_true",
                    help="measure every workload in this process. Default for 'all': the headline workload in one child "
                         "process and the others in a second one, so that no workload can cost another its measurement; "
                         "use this flag under a profiler, which must see the measuring process itself")
    ap.add_argument("--emit-results", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--variants", default="",
                    help="semicolon-separated sets of per-call library switches to time after the default configuration, "
                         "e.g. 'NMTG_GEMM_TILE=1;NMTG_ATTN_FUSED=0+NMTG_GEMM_SKINNY=0'. Each set is exported (NAME=VALUE, or NAME=1 "
                         "when no value is given) for one extra measurement of every selected workload (no CPU baseline); "
                         "results go to 'variants'.")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py measures one GPU: this build has no multi-GPU path (each op is independent per "
                         "token row / per (batch, head), so it would shard by data parallelism over tokens). Run with --gpus 1.\n")
        sys.exit(2)
    table = dict(WORKLOADS, **EXTRA_WORKLOADS)
    names = list(WORKLOADS) if args.workload == "all" else [n.strip() for n in args.workload.split(",") if n.strip()]
    if names == ["streams"]:
        names = [w.name for w in STREAM_PROBES]
    unknown = [n for n in names if n not in table]
    if unknown or not names:
        sys.stderr.write("bench.py: unknown workload %s; choose from %s\n" % (", ".join(unknown) or "''", ", ".join(table)))
        sys.exit(2)
    if PRIMARY in names:                     # headline first
        names.remove(PRIMARY)
        names.insert(0, PRIMARY)
    split = args.workload == "all" and not args.in_process and not args.variants
    variants = []
    if split:
        # This process never touches the GPU: it starts the two measuring processes and assembles their results.
        results = _in_child(names[:1], args, 900) + _in_child(names[1:], args, 2400)
        if "error" in results[0]:
            sys.stderr.write(f"bench.py: the headline workload {names[0]} gave no result: {results[0]['error']}\n")
            sys.exit(1)
    else:
        if not torch.cuda.is_available():
            sys.stderr.write("bench.py needs a GPU (MI355X); the ops have no CPU path.\n")
            sys.exit(2)
        torch.set_num_threads(os.cpu_count() or 1)
        dev = torch.device("cuda:0")
        results = _run_workloads(names, args, dev, args.emit_results)
        if args.emit_results:
            return
        # per-call switches of the library (staged kernel variants): the same workloads again under each requested set
        for spec in [v.strip() for v in args.variants.split(";") if v.strip()]:
            switches = [n.strip() for n in spec.split("+") if n.strip()]
            settings = dict((n.split("=", 1) + ["1"])[:2] for n in switches)
            saved = {n: os.environ.get(n) for n in settings}
            os.environ.update(settings)
            try:
                for n in names:
                    w = table[n]()
                    steps = args.steps if w.name not in ("xentropy", "generator_loss") else max(3, min(args.steps, 10))
                    try:
                        r = measure(w, dev, steps, args.warmup, False, min(args.trace_steps, steps))
                        variants.append(dict(switches=switches, workload=n, value=r["value"], unit=r["unit"],
                                             ms_per_step=r["ms_per_step"], kernels=r["kernels"]))
                    except Exception as e:
                        variants.append(dict(switches=switches, workload=n, error=str(e)))
                    del w
                    torch.cuda.empty_cache()
            finally:
                for n, v in saved.items():
                    if v is None:
                        os.environ.pop(n, None)
                    else:
                        os.environ[n] = v
    head = results[0]
    # The other workloads go out first, one line each, and the headline line carries only their summary: a reader of
    # the tail of this output (the last few KB) then sees every workload's figures.
    for r in results[1:]:
        print(OTHER_TAG + json.dumps(r), flush=True)

    def brief(r):
        if "error" in r:
            return dict(workload=r["workload"], error=r["error"])
        roof = r.get("roofline") or {}
        return dict(workload=r["workload"], value=r["value"], unit=r["unit"], ms_per_step=r["ms_per_step"],
                    kernel=roof.get("kernel"), frac=roof.get("frac"), traffic=roof.get("traffic"))
    line = {
        "metric": "MFMA TFLOP/s (fused MLP fwd+bwd)" if head["workload"] == "mlp" else head["metric"] + f" ({head['workload']})",
        "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": head["steps"], "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": head["dtype"], "data": head["data"],
        "config": {"workload": head["description"], "timed": head["timed"],
                   "switches": {k: v for k, v in sorted(os.environ.items()) if k.startswith("NMTG_")}},
        "roofline": head["roofline"], "cpu_baseline": head["cpu_baseline"], "kernels": head["kernels"],
        "others": [brief(r) for r in results[1:]],
    }
    if variants:
        line["variants"] = variants
    print(json.dumps(line))


if __name__ == "__main__":
    main()
