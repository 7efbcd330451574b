"""The elementwise kernels' own source, executed on the CPU.

tests/hostsim compiles layer_norm.hip, softmax_dropout.hip, dropout_add.hip and xentropy.hip (with the library's
plumbing in api.hip) as plain C++ against a small stand-in for the HIP headers and runs every kernel lane by lane:
one fiber per thread, 64-lane wavefronts that meet at shuffles, block barriers, blocks one after the other. The
resulting library exports the same extern "C" entry points as libnmtg_hip.so, so the checks below are the GPU
tests' own functions (tests/test_layer_norm_gpu.py, tests/test_elementwise_gpu.py) called with host tensors, at
sizes a CPU finishes in seconds. The compute-unit count the launch code sees is set small, so grid-stride loops make
several trips and partial last groups occur.

What this covers: indexing, masking, clamping, reduction trees, launch arithmetic, the C entry points' argument
checks. What it cannot cover: memory ordering, occupancy, anything about timing, and the GEMM / attention / MLP
kernels (MFMA, LDS transfers), which only run on the GPU.
"""
import ctypes
import itertools
import os
import subprocess
import sys

import pytest
import torch

from nmtgminor_amd import _lib, _rng

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "hostsim"))
import build as hostsim_build  # noqa: E402

import test_elementwise_gpu as tel  # noqa: E402
import test_layer_norm_gpu as tln  # noqa: E402

pytestmark = pytest.mark.skipif(not hostsim_build.available(), reason="no host C++ compiler with __bf16 (ROCm clang++)")
CPU = torch.device("cpu")
F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16


@pytest.fixture(scope="session")
def hostsim_lib():
    lib = ctypes.CDLL(hostsim_build.ensure())
    lib.nmtg_last_error.restype = ctypes.c_char_p
    lib.nmtg_version.restype = ctypes.c_int
    lib.nmtg_ln_bwd_parts.restype = ctypes.c_int64
    return lib


@pytest.fixture(autouse=True)
def on_the_cpu(hostsim_lib, monkeypatch):
    counter = itertools.count()
    monkeypatch.setattr(_lib, "_lib", hostsim_lib)                    # what _lib.load() hands out
    monkeypatch.setattr(_lib, "require_cuda", lambda *t: None)
    monkeypatch.setattr(_lib, "stream_of", lambda t: ctypes.c_void_p(0))
    monkeypatch.setenv("HOSTSIM_CUS", "2")

    # `t.to(device)` hands back a copy on the GPU box; on the CPU it would alias `t`, and the in-place operators
    # would then change the inputs the oracle is given afterwards
    plain_to = torch.Tensor.to

    def copying_to(self, *a, **k):
        out = plain_to(self, *a, **k)
        if a and isinstance(a[0], torch.device) and out.data_ptr() == self.data_ptr() and out.numel() > 0:
            out = out.clone()
        return out
    monkeypatch.setattr(torch.Tensor, "to", copying_to)

    def seed_offset(dev, n):                                          # one Philox stream, advancing like the GPU one
        return 1234, 4 * next(counter)
    for name, mod in list(sys.modules.items()):
        if name.startswith("nmtgminor_amd") and hasattr(mod, "philox_seed_offset"):
            monkeypatch.setattr(mod, "philox_seed_offset", seed_offset)


def test_only_the_simulated_operators_are_exported(hostsim_lib):
    assert hostsim_lib.nmtg_version() == 100
    with pytest.raises(AttributeError):
        hostsim_lib.nmtg_gemm


# ----------------------------------------------------------------------------- LayerNorm
@pytest.mark.parametrize("hidden", [64, 256, 768, 1024, 1536, 4096, 8192])
def test_layer_norm_hidden_sizes_fp32(hidden):
    tln._run(37, hidden, F32, F32, CPU)


@pytest.mark.parametrize("dtype,wdtype", [(F16, F16), (BF16, BF16), (F16, F32), (BF16, F32)])
@pytest.mark.parametrize("hidden", [512, 1024, 4096, 16384])
def test_layer_norm_dtype_pairs(dtype, wdtype, hidden):
    tln._run(21, hidden, dtype, wdtype, CPU)


@pytest.mark.parametrize("hidden", [2, 3, 100, 513, 1000])
def test_layer_norm_generic_kernel(hidden):
    tln._run(19, hidden, F32, F32, CPU)
    tln._run(19, hidden, BF16, BF16, CPU)


@pytest.mark.parametrize("rows", [1, 2, 3, 5, 130, 257])
def test_layer_norm_ragged_row_counts(rows):
    tln._run(rows, 512, F32, F32, CPU)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("hidden", [512, 1024, 8192])
def test_layer_norm_memory_efficient_backward(dtype, hidden):
    tln._run(45, hidden, dtype, dtype, CPU, memeff=True)


def test_layer_norm_empty_input_and_module():
    tln.test_empty_input(CPU)
    tln.test_module_and_autograd(CPU)


# ----------------------------------------------------------------------------- dropout + add
@pytest.mark.parametrize("dtype", tel.DTYPES)
@pytest.mark.parametrize("n", [1, 7, 4096, 2 * 32 * 64 + 3])
def test_dropout_add(dtype, n):
    tel.test_dropout_add_replayed_mask(CPU, dtype, n)


@pytest.mark.parametrize("dtype", tel.DTYPES)
def test_dropout_add_eval_and_wrapper(dtype):
    tel.test_dropout_add_eval_and_p0(CPU, dtype)
    tel.test_dropout_add_autograd_wrapper(CPU)


def test_dropout_add_philox_mask_matches_the_python_restatement():
    from nmtgminor_amd.native import fused_dropout_add_cuda
    n = 1 << 14
    x = torch.ones(n, dtype=BF16)
    m1, o1 = fused_dropout_add_cuda.forward(True, x.clone(), torch.zeros(n, dtype=BF16), 0.25)     # offset 0
    m2, _ = fused_dropout_add_cuda.forward(True, x.clone(), torch.zeros(n, dtype=BF16), 0.25)      # offset 4
    assert not torch.equal(m1, m2)
    assert abs(m1.float().mean().item() - 0.75) < 2e-2
    for first in (0, 4, 1000, n - 16):
        assert m1[first:first + 16].tolist() == _rng.philox_keep_mask_reference(1234, 0, first, 16, 0.75)
        assert m2[first:first + 16].tolist() == _rng.philox_keep_mask_reference(1234, 4, first, 16, 0.75)


# ----------------------------------------------------------------------------- masked softmax (+ dropout)
@pytest.mark.parametrize("dtype", tel.DTYPES)
@pytest.mark.parametrize("bh,tq,tk", [(8, 9, 56), (6, 5, 1), (4, 6, 512), (4, 3, 1500), (2, 16, 128), (2, 3, 2048),
                                      (4, 7, 333), (2, 2, 4096)])
def test_softmax_dropout(dtype, bh, tq, tk):
    if tk == 4096 and dtype == F32:
        pytest.skip("4096 keys is the 16-bit limit")
    tel.test_softmax_dropout_fwd_bwd(CPU, dtype, bh, tq, tk)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_softmax_time_mask_and_empty_rows(dtype):
    tel.test_softmax_time_mask_premasked_scores_and_empty_rows(CPU, dtype)


# ----------------------------------------------------------------------------- cross-entropy
@pytest.mark.parametrize("dtype", tel.DTYPES)
@pytest.mark.parametrize("n,v", [(12, 32320), (5, 7), (3, 1), (17, 4099), (6, 250054 // 8 + 1)])
def test_xentropy(dtype, n, v):
    tel._xent_case(CPU, n, v, dtype, 0.1, pad=0)


@pytest.mark.parametrize("misalign", [1, 3, 5])
def test_xentropy_misaligned_base(misalign):
    tel._xent_case(CPU, 9, 1001, BF16, 0.1, pad=0, misalign=misalign)


def test_xentropy_no_smoothing_module_and_autograd():
    tel.test_xentropy_no_smoothing_and_module_parity(CPU)
    tel.test_xentropy_autograd_function(CPU)


# ----------------------------------------------------------------------------- reductions that follow a GEMM
CODE = {F32: 0, F16: 1, BF16: 2}


@pytest.mark.parametrize("dtype", tel.DTYPES)
@pytest.mark.parametrize("m,n,pad", [(1, 8, 0), (7, 40, 0), (128, 256, 8), (129, 24, 0), (1000, 264, 0), (8195, 64, 8),
                                     (2100, 37, 3), (16, 1, 0), (4099, 520, 0)])
def test_column_sums(hostsim_lib, dtype, m, n, pad):
    # small integers: every partial sum is exact in fp32, so each row must be counted exactly once
    g = torch.Generator().manual_seed(61)
    ld = n + pad
    x = torch.randint(-8, 9, (m, ld), generator=g).to(dtype)
    parts = hostsim_lib.hostsim_colsum_parts(m)
    part = torch.full((parts, n), float("nan"))
    out = torch.full((n,), float("nan"), dtype=dtype)
    rc = hostsim_lib.hostsim_colsum(CODE[dtype], ctypes.c_void_p(x.data_ptr()), ctypes.c_int64(ld), m, n,
                                    ctypes.c_void_p(part.data_ptr()), ctypes.c_void_p(out.data_ptr()))
    assert rc == 0
    want = x[:, :n].double().sum(0)
    assert torch.equal(part.double().sum(0), want)
    assert torch.equal(out, want.to(dtype))


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("tile,m,n,batch,splits,c_vec", [(1, 128, 128, 1, 4, 8), (1, 200, 136, 2, 5, 8), (1, 77, 50, 1, 3, 1),
                                                         (0, 256, 256, 1, 8, 8), (0, 300, 260, 1, 11, 4), (1, 128, 128, 3, 1, 8)])
def test_split_k_reduction(hostsim_lib, dtype, tile, m, n, batch, splits, c_vec):
    bm, bn, wm, wn = (128, 128, 2, 2) if tile == 1 else (256, 256, 2, 4)
    wtm, wtn = bm // wm, bn // wn
    tm, tn = wtm // 32, wtn // 32
    m_tiles, n_tiles = -(-m // bm), -(-n // bn)
    per_blk = wm * wn * tm * tn * 4 * 64                       # 4-float slots per tile, in accumulator order
    total = batch * m_tiles * n_tiles * per_blk
    g = torch.Generator().manual_seed(62)
    ws = torch.randint(-16, 17, (splits, total, 4), generator=g).float()
    ldc = n + 8
    c = torch.full((batch, m, ldc), 777.0).to(dtype)
    rc = hostsim_lib.hostsim_splitk_reduce(CODE[dtype], tile, ctypes.c_void_p(ws.data_ptr()), ctypes.c_void_p(c.data_ptr()),
                                           ctypes.c_int64(ldc), m, n, m_tiles, n_tiles, batch, ctypes.c_int64(m * ldc), splits,
                                           ctypes.c_float(0.5), c_vec)
    assert rc == 0
    # slot -> (row, first column): lane, quad, column fragment, row fragment, wavefront, tile, batch entry
    idx = torch.arange(total)
    lane, t = idx & 63, idx >> 6
    q, t = t & 3, t >> 2
    j, t = t % tn, t // tn
    i, t = t % tm, t // tm
    wave, t = t % (wm * wn), t // (wm * wn)
    tile_id, bz = t % (m_tiles * n_tiles), t // (m_tiles * n_tiles)
    row = (tile_id // n_tiles) * bm + (wave // wn) * wtm + i * 32 + (lane & 31)
    col = (tile_id % n_tiles) * bn + (wave % wn) * wtn + j * 32 + q * 8 + (lane >> 5) * 4
    want = torch.full((batch, m, ldc), 777.0, dtype=torch.float64)
    summed = ws.double().sum(0) * 0.5
    for e in range(4):
        ok = (row < m) & (col + e < n)
        want[bz[ok], row[ok], col[ok] + e] = summed[ok, e]
    assert torch.equal(c.double(), want.to(dtype).double())
    assert (want[:, :, :n] != 777.0).all()                      # every element of C has exactly one slot


# ----------------------------------------------------------------------------- the same checks, bounds-checked
def test_every_check_again_under_address_sanitizer():
    """A child process repeats this file against an AddressSanitizer build of the same sources, with the sanitizer's
    runtime preloaded: PyTorch's host allocations then carry red zones, and any kernel load or store outside the
    tensor it was handed (a clamped index that is not clamped, a vector access across the end of a row) stops the run
    with the kernel's file and line."""
    if os.environ.get("HOSTSIM_SANITIZE") == "1":
        pytest.skip("this is the sanitizer run")
    preloaded = os.environ.get("LD_PRELOAD", "").strip()
    if os.path.exists("/etc/ld.so.preload"):
        with open("/etc/ld.so.preload") as f:
            preloaded += f.read().strip()
    if preloaded:
        pytest.skip("another library is preloaded; the sanitizer's runtime has to come first")
    runtime = subprocess.run([hostsim_build.CXX, "-print-file-name=libclang_rt.asan-x86_64.so"], capture_output=True,
                             text=True).stdout.strip()
    if not os.path.isabs(runtime) or not os.path.exists(runtime):
        pytest.skip("no AddressSanitizer runtime beside the compiler")
    env = dict(os.environ, HOSTSIM_SANITIZE="1", LD_PRELOAD=runtime,
               ASAN_OPTIONS="detect_leaks=0:detect_stack_use_after_return=0")
    run = subprocess.run([sys.executable, "-m", "pytest", os.path.abspath(__file__), "-x", "-q", "-p", "no:cacheprovider"],
                         env=env, capture_output=True, text=True, timeout=1500,
                         cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert run.returncode == 0, (run.stdout[-3000:] + run.stderr[-3000:])
