"""The kernels' own source, executed on the CPU.

tests/hostsim compiles the library's .hip sources as plain C++ against a small stand-in for the HIP headers and runs
every kernel lane by lane: one fiber per thread, 64-lane wavefronts that meet at shuffles, MFMA instructions and LDS
transpose reads, block barriers, blocks one after the other; the asynchronous global -> LDS transfers of the GEMM
loops land either as late or as early as the kernel's own waits allow (HOSTSIM_DMA). The resulting library exports
the same extern "C" entry points as libnmtg_hip.so, so the checks below are the GPU tests' own functions
(tests/test_*_gpu.py) called with host tensors, at sizes a CPU finishes in seconds.

What this covers: indexing, masking, clamping, LDS layouts and fragment reads, reduction trees, launch arithmetic,
tile selection, workspace use, the waits that order LDS transfers against their reads, the C entry points' argument
checks, and (in the sanitizer run at the end) that no kernel touches memory outside the tensors it was handed.
What it cannot cover: real memory ordering and caches, occupancy, register pressure, anything about speed. A GPU
run of the same tests remains the proof; this run keeps mistakes of the first kind from ever reaching the GPU.
"""
import ctypes
import os
import subprocess
import sys
import tempfile

import pytest
import torch

from nmtgminor_amd import _rng

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "hostsim"))
import harness  # noqa: E402
from harness import hostsim_build  # noqa: E402

import test_attention_gpu as tat  # noqa: E402
import test_elementwise_gpu as tel  # noqa: E402
import test_gemm_gpu as tg  # noqa: E402
import test_layer_norm_gpu as tln  # noqa: E402
import test_zu_random_shapes_gpu as trnd  # noqa: E402
import test_zv_empty_inputs_gpu as temp  # noqa: E402
import test_zw_strided_inputs_gpu as tstr  # noqa: E402
import test_zx_incremental_gpu as tinc  # noqa: E402
import test_zy_layers_gpu as tla  # noqa: E402
import test_mlp_gpu as tm  # noqa: E402
import test_kernel_variants_gpu as tst  # noqa: E402
import test_zz_golden_gpu as tgold  # noqa: E402
import test_zzb_generator_loss_gpu as tgen  # noqa: E402
import test_zzc_relative_attention_gpu as trel  # noqa: E402
import test_zzd_fused_optim_gpu as topt  # noqa: E402
import test_zze_flash_attention_gpu as tfl  # noqa: E402
import test_zzf_feed_forward_gpu as tff  # noqa: E402
import test_zzg_attention_no_coverage_gpu as tnc  # noqa: E402

pytestmark = pytest.mark.skipif(not hostsim_build.available(), reason="no host C++ compiler with __bf16 (ROCm clang++)")
CPU = torch.device("cpu")
F32, F16, BF16 = torch.float32, torch.float16, torch.bfloat16
SANITIZER_RUN = os.environ.get("HOSTSIM_SANITIZE") == "1"
# the sanitizer build is several times slower: it repeats every check except the ones marked long
long_case = pytest.mark.skipif(SANITIZER_RUN, reason="left out of the sanitizer run for time")
HALVES = [BF16] if SANITIZER_RUN else [F16, BF16]          # the two 16-bit types share every index computation


_sanitizer_run = {}

_SANITIZER_CHILD = """
import os, subprocess, sys
build, test_file, runtime, log = sys.argv[1:5]
env = dict(os.environ, HOSTSIM_SANITIZE="1")
rc = subprocess.run([sys.executable, build, "--if-stale"], env=env, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL).returncode
if rc == 0:
    env.update(LD_PRELOAD=runtime, ASAN_OPTIONS="detect_leaks=0:detect_stack_use_after_return=0", OMP_NUM_THREADS="2")
    spread = []          # the checks are independent of each other: four worker processes where pytest-xdist is there
    try:
        import xdist
        spread = ["-n", "4"]
    except ImportError:
        pass
    with open(log, "w") as out:
        rc = subprocess.run([sys.executable, "-m", "pytest", test_file, "-x", "-q", "-p", "no:cacheprovider"] + spread, env=env,
                            stdout=out, stderr=subprocess.STDOUT, cwd=os.path.dirname(os.path.dirname(test_file))).returncode
sys.exit(rc)
"""


def _start_sanitizer_run():
    """Starts, beside this process, the child that builds the AddressSanitizer variant of the kernels and repeats this
    file against it (the last test of the file collects its result). -> reason for not running it, or None."""
    preloaded = os.environ.get("LD_PRELOAD", "").strip()
    if os.path.exists("/etc/ld.so.preload"):
        with open("/etc/ld.so.preload") as f:
            preloaded += f.read().strip()
    if preloaded:
        return "another library is preloaded; the sanitizer's runtime has to come first"
    runtime = subprocess.run([hostsim_build.CXX, "-print-file-name=libclang_rt.asan-x86_64.so"], capture_output=True,
                             text=True).stdout.strip()
    if not os.path.isabs(runtime) or not os.path.exists(runtime):
        return "no AddressSanitizer runtime beside the compiler"
    log = tempfile.NamedTemporaryFile(prefix="hostsim_asan_", suffix=".log", delete=False)
    log.close()
    _sanitizer_run["log"] = log.name
    _sanitizer_run["proc"] = subprocess.Popen([sys.executable, "-c", _SANITIZER_CHILD, os.path.join(harness.HERE, "hostsim_build.py"),
                                               os.path.abspath(__file__), runtime, log.name])
    return None


@pytest.fixture(scope="session")
def hostsim_lib():
    lib = harness.library()
    if not SANITIZER_RUN and "skip" not in _sanitizer_run and "proc" not in _sanitizer_run:
        _sanitizer_run["skip"] = _start_sanitizer_run()
    return lib


@pytest.fixture(autouse=True)
def on_the_cpu(hostsim_lib, monkeypatch):
    harness.install(monkeypatch.setattr)
    # elementwise kernels: few compute units, so that grid-stride loops make several trips and last groups are partial
    monkeypatch.setenv("HOSTSIM_CUS", "2")
    monkeypatch.delenv("HOSTSIM_DMA", raising=False)
    # products with few rows stay on the tiled kernels here (the few-row kernel has its own test below), so that the
    # layers' small test shapes keep exercising the tiled kernels' edge handling
    monkeypatch.setenv("NMTG_GEMM_SKINNY", "0")


@pytest.fixture
def mi355x(monkeypatch):
    """GEMM-based operators: the tile and split-K choices depend on the compute-unit count, so show them the real one."""
    monkeypatch.setenv("HOSTSIM_CUS", "256")


@pytest.fixture(params=["late", "early"])
def dma(request, monkeypatch):
    monkeypatch.setenv("HOSTSIM_DMA", request.param)
    return request.param


def test_every_entry_point_is_exported(hostsim_lib):
    # the tracing pair counts launches per kernel name here (no HIP events to time)
    from nmtgminor_amd import _lib
    assert hostsim_lib.nmtg_version() == 100
    missing = [n for n in _lib.header_functions() if not hasattr(hostsim_lib, n)]
    assert missing == []


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


@long_case
def test_xentropy_no_smoothing_module_and_autograd():
    tel.test_xentropy_no_smoothing_and_module_parity(CPU)
    tel.test_xentropy_autograd_function(CPU)


# ----------------------------------------------------------------------------- reductions that follow a GEMM
CODE = {F32: 0, F16: 1, BF16: 2}


@pytest.mark.parametrize("nbytes", [16, 4096 * 16 + 48])
def test_streaming_probes(nbytes):
    tel.test_streaming_probes_move_what_they_say(CPU, nbytes)


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


# ----------------------------------------------------------------------------- GEMM core
@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (128, 128, 128), (300, 200, 72), (1, 8, 8), (257, 129, 1000), (64, 1504, 64),
                                   pytest.param(512, 2048, 512, marks=long_case), pytest.param(1024, 64, 512, marks=long_case)])
@pytest.mark.parametrize("layout", ["nt", "nn", "tn"])
def test_gemm_layouts(mi355x, dtype, m, n, k, layout):
    tg.test_gemm_layouts(CPU, dtype, m, n, k, layout)


@pytest.mark.parametrize("layout", ["nt", "nn", "tn"])
@pytest.mark.parametrize("m,n,k", [(300, 520, 448), (700, 130, 256)])
def test_gemm_ring_under_both_transfer_timings(mi355x, dma, layout, m, n, k):
    # K of several 64-steps: the ring wraps around, slots are refilled while later wavefronts still read
    tg.test_gemm_layouts(CPU, BF16, m, n, k, layout)


@long_case
@pytest.mark.parametrize("dtype", HALVES)
def test_gemm_unaligned_extents(mi355x, dtype):
    tg.test_gemm_unaligned_extents(CPU, dtype)


def test_gemm_bias_and_batched_strided_views(mi355x):
    tg.test_gemm_bias_and_batched_strided_views(CPU)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("v", [1030, 70, 6])
def test_gemm_ragged_extents_on_aligned_operands(mi355x, dma, dtype, v):
    # also asserts which kernels ran: 16-byte accesses throughout, the slot-ring loop where the reduction allows it
    tg.test_ragged_extents_keep_16_byte_accesses(CPU, dtype, v)


def test_gemm_transposed_product_without_workspace(mi355x):
    tg.test_transposed_product_without_workspace_runs_unsplit(CPU)


@long_case
def test_gemm_split_k(mi355x, hostsim_lib):
    # reduction-heavy dW-shaped product: the call splits K and reduces the partials in a fixed order
    m, n, k = 256, 128, 4096
    assert hostsim_lib.nmtg_gemm_workspace_bytes(ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k), ctypes.c_int64(1)) > 0
    a, b = tg._mk((k, m), CPU, F16, 11), tg._mk((k, n), CPU, F16, 12)
    c1, c2 = tg.gemm(a, b, True, False), tg.gemm(a, b, True, False)
    assert torch.equal(c1, c2)
    tg.assert_close(c1, tg._ref(a, b, True, False), F16, "split-k", scale_atol=True)
    tg.assert_close(tg.gemm(a, b, True, False, split_k=False), tg._ref(a, b, True, False), F16, "no split", scale_atol=True)


# ----------------------------------------------------------------------------- fused MLP
@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("act", ["gelu", "relu", "silu", "agelu"])
@pytest.mark.parametrize("tokens,dm,di,p", [(72, 96, 200, 0.5), pytest.param(256, 128, 256, 0.0, marks=long_case)])
def test_mlp_autograd_function(mi355x, dtype, act, tokens, dm, di, p):
    tm.test_mlp_autograd_function(CPU, dtype, act, tokens, dm, di, p)


@long_case
def test_mlp_recompute_input_only_three_layers_rng(mi355x):
    tm.test_mlp_recompute_and_input_only(CPU)
    tm.test_mlp_three_layers_and_rng_mask(CPU)


# ----------------------------------------------------------------------------- attention
@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("t,b,e,h,p", [pytest.param(64, 4, 256, 4, 0.0, marks=long_case), (33, 2, 128, 2, 0.1),
                                       pytest.param(200, 2, 256, 4, 0.25, marks=long_case)])
def test_self_attention_key_padding(mi355x, dtype, t, b, e, h, p):
    tat.test_self_attention_key_padding(CPU, dtype, t, b, e, h, p)


@long_case
def test_self_attention_contract_rng_eval_no_bias(mi355x):
    tat.test_self_attention_intermediates_and_native_contract(CPU)
    tat.test_self_attention_rng_dropout_eval_and_no_bias(CPU)


@long_case
def test_self_attention_causal_and_recompute(mi355x):
    tat.test_self_attention_causal_and_recompute(CPU, BF16)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("tq,tk,b,e,h,p", [(17, 100, 3, 128, 2, 0.2), pytest.param(32, 1500, 2, 256, 4, 0.1, marks=long_case)])
def test_encdec_attention(mi355x, dtype, tq, tk, b, e, h, p):
    tat.test_encdec_attention(CPU, dtype, tq, tk, b, e, h, p)


@long_case
@pytest.mark.parametrize("split", ["0", "1"])
def test_attention_inference_without_the_score_tensor(mi355x, monkeypatch, split):
    tat.test_self_attention_inference_without_the_score_tensor(CPU, monkeypatch, BF16, 100, 3, 256, 4, False, split)
    tat.test_self_attention_inference_without_the_score_tensor(CPU, monkeypatch, F16, 72, 2, 256, 2, True, split)
    tat.test_encdec_attention_inference_without_the_score_tensor(CPU, monkeypatch, BF16, 17, 100, 3, 128, 2, True, split)
    tat.test_encdec_attention_inference_without_the_score_tensor(CPU, monkeypatch, F16, 5, 260, 1, 128, 1, True, split)
    tat.test_inference_without_coverage_writes_no_probability_tensor(CPU, monkeypatch, split)
    tat.test_inference_keeps_the_score_tensor_where_the_one_kernel_path_does_not_apply(CPU, monkeypatch)   # sets a switch: last


@pytest.mark.parametrize("seed", [4000, 4003, 4005, 4008] if SANITIZER_RUN else list(range(4000, 4012)))
def test_attention_inference_random_shapes(mi355x, monkeypatch, seed):
    tat.test_inference_kernel_on_randomly_drawn_shapes(CPU, monkeypatch, seed)


@pytest.mark.parametrize("mode", ["eval", "eval_no_coverage", "recompute_p0"])
def test_self_attention_backward_without_dropout_state(mi355x, mode):
    tat.test_self_attention_backward_without_dropout_state(CPU, mode)


@pytest.mark.parametrize("mode", ["eval", "eval_compact", "recompute_p0"])
def test_encdec_attention_backward_without_dropout_state(mi355x, mode):
    tat.test_encdec_attention_backward_without_dropout_state(CPU, mode)


def test_encdec_attention_without_biases_compact_and_modules(mi355x):
    tat.test_encdec_attention_without_biases_and_compact(CPU)
    tat.test_modules_state_dict_names_and_forward(CPU)
    tat.test_feed_forward_module(CPU)


# ----------------------------------------------------------------------------- layer glue
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_pre_post_processing(mi355x, dtype):
    tla.test_pre_post_processing_sequences(CPU, dtype)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("macaron,training", [pytest.param(False, False, marks=long_case), pytest.param(False, True, marks=long_case),
                                              (True, True)])
def test_encoder_layer(mi355x, dtype, macaron, training):
    tla.test_encoder_layer_matches_the_oracle(CPU, dtype, macaron, training)


def test_encoder_layer_on_the_tiled_attention_core(mi355x, monkeypatch):
    tla.test_encoder_layer_with_head_dimension_64_drops_the_coverage_and_runs_the_tiled_core(CPU, BF16, monkeypatch)


@long_case
def test_decoder_layer_on_the_tiled_attention_core(mi355x, monkeypatch):
    tla.test_decoder_layer_with_head_dimension_64_runs_its_self_attention_on_the_tiled_core(CPU, F16, monkeypatch)


@pytest.mark.parametrize("dtype", HALVES)
def test_training_attention_with_time_masks_without_coverage(mi355x, dtype):
    if not SANITIZER_RUN:
        tnc.test_self_attention_training_with_a_causal_time_mask(CPU, dtype, 200, 2, 256, 4, 0.25)
    tnc.test_self_attention_training_with_time_masks_of_other_shapes(CPU, dtype)
    tnc.test_a_causal_time_mask_equals_the_causal_flag_bit_for_bit(CPU, 64, 0.2)


@pytest.mark.parametrize("order", ["reverse", "interleave_random"])
def test_tiled_kernels_do_not_depend_on_the_order_of_their_wavefronts(mi355x, monkeypatch, order):
    """Between two block barriers the wavefronts of a block may run in any order and interleaving: the tiled attention
    kernels with a time mask (bit for bit against the causal flag) and the ring GEMM give the same results when the
    CPU build runs them last-to-first, or one wavefront-wide operation at a time in a random order."""
    monkeypatch.setenv("HOSTSIM_ORDER", order)
    monkeypatch.setenv("HOSTSIM_SEED", "11")
    tnc.test_a_causal_time_mask_equals_the_causal_flag_bit_for_bit(CPU, 64, 0.2)
    tnc.test_self_attention_training_with_time_masks_of_other_shapes(CPU, BF16)
    tg.test_gemm_layouts(CPU, F16, 300, 520, 448, "nn")


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("ignore_source", [False, pytest.param(True, marks=long_case)])
def test_decoder_layer(mi355x, dtype, ignore_source):
    tla.test_decoder_layer_matches_the_oracle(CPU, dtype, ignore_source)


@long_case
def test_layers_stochastic_depth_dropout_and_options(mi355x):
    tla.test_encoder_layer_stochastic_depth(CPU)
    tla.test_layers_with_dropout_and_unsupported_options(CPU)


# ----------------------------------------------------------------------------- randomly drawn shapes
@pytest.mark.parametrize("seed", trnd.SEEDS[:16] if SANITIZER_RUN else trnd.SEEDS)
def test_random_shapes(mi355x, seed):
    trnd.test_random_shape(CPU, seed)


# ----------------------------------------------------------------------------- empty inputs
@pytest.mark.parametrize("name", [n for n in dir(temp) if n.startswith("test_")])
def test_empty_inputs(mi355x, name):
    getattr(temp, name)(CPU)


# ----------------------------------------------------------------------------- strided arguments
@pytest.mark.parametrize("name", [n for n in dir(tstr) if n.startswith("test_") and "row_pitched" not in n and "slice_of" not in n])
def test_strided_arguments(mi355x, name):
    getattr(tstr, name)(CPU)


@pytest.mark.parametrize("dtype", [BF16, torch.float32])
def test_cross_entropy_backward_on_a_slice_of_the_classes(mi355x, dtype):
    tstr.test_cross_entropy_backward_on_a_slice_of_the_classes(CPU, dtype)


@pytest.mark.parametrize("dtype", [F16, torch.float32])
@pytest.mark.parametrize("v,pitch,gpitch", [(1000, 1024, 1024), (517, 520, 576), (250, 251, 250)])
def test_cross_entropy_on_row_pitched_logits(mi355x, dtype, v, pitch, gpitch):
    tstr.test_cross_entropy_reads_and_writes_row_pitched_logits_in_place(CPU, dtype, v, pitch, gpitch)


# ----------------------------------------------------------------------------- incremental decoding
@pytest.mark.parametrize("dtype", HALVES)
def test_incremental_decoding(mi355x, dtype):
    tinc.test_self_attention_step_by_step(CPU, dtype, 3)
    tinc.test_self_attention_steps_honour_a_key_padding_mask(CPU, dtype)
    tinc.test_cross_attention_with_cached_encoder_states(CPU, dtype)


@pytest.mark.parametrize("d", [32, 64, 128])
def test_decoding_kernel_skips_the_padded_tail_of_the_cache(d):
    tinc.test_one_position_does_not_read_the_cache_behind_a_sentences_last_live_key(CPU, d)


@long_case
def test_incremental_decoder_layer_with_beam_reordering(mi355x):
    tinc.test_self_attention_step_by_step(CPU, F16, 1)
    tinc.test_decoder_layer_step_by_step_with_beam_reordering(CPU)


# ----------------------------------------------------------------------------- projection + loss in row chunks
@pytest.mark.parametrize("dtype", HALVES)
def test_chunked_projection_loss(mi355x, dtype):
    tgen.test_chunked_projection_loss_matches_oracle_and_unchunked_operators(CPU, dtype, 40, 64, 250, 16, True, 0.1, True)
    if not SANITIZER_RUN:
        tgen.test_chunked_projection_loss_matches_oracle_and_unchunked_operators(CPU, dtype, 80, 64, 1000, 32, True, 0.1, False)
        tgen.test_chunked_projection_loss_matches_oracle_and_unchunked_operators(CPU, dtype, 33, 64, 2048, 8, True, 0.3, True)


@long_case
def test_chunked_projection_loss_module_and_validation(mi355x):
    tgen.test_chunked_projection_loss_matches_oracle_and_unchunked_operators(CPU, F16, 64, 128, 517, 64, False, 0.0, False)
    tgen.test_per_row_weights_and_no_gradient_for_frozen_weights(CPU)
    tgen.test_validation_pass_counts_correct_predictions(CPU)
    tgen.test_module_matches_the_reference_loss_assembly(CPU)
    tgen.test_argument_checks_and_empty_batch(CPU)


# ----------------------------------------------------------------------------- relative-position self-attention
@pytest.mark.parametrize("dtype", [BF16, F16, F32])
@pytest.mark.parametrize("b,tq,tk,r", [(3, 16, 16, 16), (2, 9, 9, 13), (1, 40, 40, 48), (2, 7, 5, 8), (1, 1, 1, 1)])
def test_relative_shift_kernels(mi355x, dtype, b, tq, tk, r):
    trel.test_shift_add_and_its_adjoint_move_values_exactly(CPU, dtype, b, tq, tk, r)


@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("bh,heads,tq,tk,r,mask,p", [(4, 2, 24, 24, 40, "pad", 0.25), (2, 1, 40, 16, 16, "time", 0.25),
                                                     (2, 2, 5, 1032, 1032, None, 0.1), (3, 1, 1, 8, 8, None, 0.0)])
def test_relative_shift_folded_into_the_softmax(mi355x, dtype, bh, heads, tq, tk, r, mask, p):
    trel.test_shift_folded_into_the_softmax_matches_the_separate_kernels(CPU, dtype, bh, heads, tq, tk, r, mask, p)
    trel.test_fused_shift_is_refused_for_rows_the_wide_kernels_cannot_take(CPU)


def test_relative_position_elementwise_kernels_and_linear_layer(mi355x):
    trel.test_shift_refuses_fewer_positions_than_keys(CPU)
    for t, b, h, d in ((5, 2, 4, 64), (3, 1, 3, 20), (4, 2, 2, 7)):
        for dtype in (BF16, F32):
            trel.test_query_bias_adds_per_head_biases_to_queries_inside_the_projection(CPU, dtype, t, b, h, d)
    for rows, cols, pitch in ((300, 64, 64), (129, 40, 48), (5, 7, 7), (1000, 520, 1024), (1, 16, 16)):
        for dtype in (BF16, F16, F32):
            trel.test_column_sums(CPU, dtype, rows, cols, pitch)
    trel.test_linear_layer_and_its_three_gradients(CPU, BF16)
    trel.test_linear_module_and_frozen_weight(CPU, True)
    trel.test_linear_module_and_frozen_weight(CPU, False)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("t,b,e,h,len_r,pos_batch,causal,p", [
    (64, 2, 256, 4, None, 1, False, 0.1), pytest.param(48, 3, 128, 2, 80, 1, False, 0.0, marks=long_case),
    (40, 2, 128, 4, None, 2, True, 0.25), (33, 1, 192, 3, 37, 1, False, 0.1)])
def test_relative_attention(mi355x, dtype, t, b, e, h, len_r, pos_batch, causal, p):
    trel.test_relative_attention_matches_oracle(CPU, dtype, t, b, e, h, len_r, pos_batch, causal, p)


def test_relative_attention_module_and_inference(mi355x):
    trel.test_inference_returns_probabilities_and_single_output_form(CPU)
    trel.test_module_has_the_reference_parameters_and_runs(CPU)
    trel.test_module_with_learnable_positions(CPU)
    trel.test_empty_batch_gives_empty_results_and_zero_parameter_gradients(CPU, 0, 2)
    trel.test_empty_batch_gives_empty_results_and_zero_parameter_gradients(CPU, 5, 0)
    trel.test_extension_stand_in_keeps_the_reference_argument_order_and_lists(CPU)
    trel.test_step_by_step_decoding_reproduces_the_causal_rows(CPU)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("t,b,e,h,causal,p", [(48, 2, 128, 2, False, 0.1), (33, 3, 192, 3, True, 0.0)])
def test_relative_attention_with_learnable_positions(mi355x, dtype, t, b, e, h, causal, p):
    trel.test_learnable_position_attention_matches_oracle(CPU, dtype, t, b, e, h, causal, p)


@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("shape,view", [((6, 8, 3, 16), "queries"), ((40, 24), "dense"), ((5, 7), "odd"), ((0, 8), "empty")])
def test_row_add(mi355x, dtype, shape, view):
    trel.test_row_add_on_dense_and_pitched_rows(CPU, dtype, shape, view)


# ----------------------------------------------------------------------------- multi-tensor optimizer passes
@pytest.mark.parametrize("dtype", [F32, BF16, pytest.param(F16, marks=long_case)])
@pytest.mark.parametrize("mode,bias_correction,wd", [(1, 1, 0.01), pytest.param(0, 1, 0.01, marks=long_case),
                                                     pytest.param(1, 0, 0.0, marks=long_case)])
def test_multi_tensor_adam(dtype, mode, bias_correction, wd):
    topt.test_adam_update_of_a_list_of_tensors(CPU, dtype, mode, bias_correction, wd)


def test_multi_tensor_scale_and_norm():
    topt.test_adam_argument_checks(CPU)
    # the sanitizer run repeats one dtype pair of each pass: the index arithmetic is the same for all of them
    for src, dst in ((F16, F32),) if SANITIZER_RUN else ((F32, F32), (F16, F32), (F32, BF16), (BF16, BF16)):
        topt.test_scale_with_overflow_flag(CPU, src, dst)
    for dtype in (BF16,) if SANITIZER_RUN else (F32, BF16, F16):
        topt.test_l2norm_of_a_list_of_tensors(CPU, dtype)
    for max_norm in (0.5,) if SANITIZER_RUN else (0.5, 1e6, 0.0):
        topt.test_clip_grad_norm_matches_torch(CPU, max_norm)
    for a, b in ((F16, F32),) if SANITIZER_RUN else ((F32, F32), (F16, F32), (BF16, BF16)):
        topt.test_axpby_with_overflow_check(CPU, a, b)
        topt.test_l2norm_with_scaling_in_one_pass(CPU, a, b)


@pytest.mark.parametrize("seed", [3000] + [pytest.param(s, marks=long_case) for s in (3001, 3002, 3003, 3004)])
def test_multi_tensor_random_lists(seed):
    topt.test_randomly_drawn_tensor_lists(CPU, seed)


@pytest.mark.parametrize("seed", [2000, 2001, 2002] + [pytest.param(s, marks=long_case) for s in range(2003, 2008)])
def test_relative_position_random_shapes(mi355x, seed):
    trel.test_randomly_drawn_shapes(CPU, seed)


@pytest.mark.parametrize("dtype,adam_w", [(F32, True), (F32, False), (BF16, True)])
def test_fused_adam_optimizer(dtype, adam_w):
    topt.test_fused_adam_follows_torch_adamw(CPU, dtype, adam_w)


# ----------------------------------------------------------------------------- default paths against the plainer ones their diagnostic switches select
@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("batch,m,n,k", [(3, 300, 64, 192), (2, 256, 64, 64), (5, 77, 64, 128)])
def test_ring_loop_of_the_256x64_tile(mi355x, dma, dtype, batch, m, n, k):
    tst.test_ring_256x64_products(CPU, dtype, batch, m, n, k)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("t,b,e,h,p,causal", [pytest.param(200, 2, 256, 4, 0.25, False, marks=long_case), (96, 2, 128, 2, 0.1, True),
                                              (40, 2, 128, 2, 0.1, False), pytest.param(512, 2, 256, 4, 0.1, False, marks=long_case)])
def test_fused_scores_softmax(mi355x, dtype, t, b, e, h, p, causal):
    tst.test_fused_scores_softmax_matches_two_kernel_path(CPU, dtype, t, b, e, h, p, causal)


def test_fused_scores_softmax_draws_the_same_dropout_mask(mi355x):
    tst.test_fused_scores_softmax_rng_mask_is_the_same_stream(CPU)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("t,b,e,h,p,causal", [pytest.param(96, 2, 128, 2, 0.0, True, marks=long_case), (40, 2, 128, 2, 0.1, False),
                                              pytest.param(200, 2, 256, 4, 0.25, False, marks=long_case)])
def test_fused_softmax_backward(mi355x, dtype, t, b, e, h, p, causal):
    tst.test_fused_softmax_backward_matches_two_kernel_path(CPU, dtype, t, b, e, h, p, causal)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("tokens,dm,di,p", [(256, 128, 256, 0.1), pytest.param(300, 192, 448, 0.0, marks=long_case)])
def test_table_gelu(mi355x, dtype, tokens, dm, di, p):
    tst.test_table_gelu_matches_the_formula(CPU, dtype, tokens, dm, di, p)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("tq,tk,b,e,h,masked", [(17, 100, 3, 128, 2, True), (8, 70, 2, 128, 2, False),
                                                pytest.param(32, 1500, 2, 256, 4, True, marks=long_case)])
def test_padded_keys(mi355x, dtype, tq, tk, b, e, h, masked):
    # also the regression test for saved tensors that reach the backward as non-contiguous views
    tst.test_padded_keys_give_the_same_cross_attention(CPU, dtype, tq, tk, b, e, h, masked)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("tokens,dm,di", [pytest.param(4096, 128, 256, marks=long_case), pytest.param(1000, 192, 448, marks=long_case),
                                          (300, 64, 128)])
def test_mlp_backward_with_one_reduction_launch(mi355x, dtype, tokens, dm, di):
    tst.test_mlp_backward_with_one_reduction_launch(CPU, dtype, tokens, dm, di)


@long_case
def test_three_layer_mlp_backward_with_one_reduction_launch(mi355x):
    tst.test_three_layer_mlp_backward_with_one_reduction_launch(CPU)


# ----------------------------------------------------------------------------- attention over packed sequences
@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("d,causal", [(64, False), (64, True), pytest.param(128, True, marks=long_case)])
def test_packed_attention_ragged(dtype, d, causal):
    tfl.test_ragged_self_attention_matches_the_oracle(CPU, dtype, d, causal)


def test_packed_attention_unequal_lengths_and_empty_sequences():
    tfl.test_different_query_and_key_lengths_and_an_empty_sequence(CPU, BF16)


@pytest.mark.parametrize("dtype,d,causal", [(BF16, 64, True), pytest.param(F16, 128, False, marks=long_case)])
def test_packed_attention_dropout_replay(dtype, d, causal):
    tfl.test_dropout_with_a_replayed_mask(CPU, dtype, d, causal)


def test_packed_attention_dropout_philox_and_autograd_functions():
    tfl.test_dropout_drawn_on_the_device_is_the_documented_philox_stream_in_both_passes(CPU, F16, 64)
    tfl.test_packed_qkv_function_takes_strided_slots_and_fills_one_gradient_tensor(CPU, BF16)
    tfl.test_packed_kv_function_with_dropout_repeats_its_mask_in_the_backward(CPU)


# ----------------------------------------------------------------------------- the same kernels over a padded batch
def test_training_attention_without_coverage(mi355x, monkeypatch):
    tnc.test_self_attention_with_masked_keys_anywhere(CPU, BF16)
    tnc.test_encdec_attention_training_without_coverage(CPU, F16, 17, 100, 3, 128, 2, 0.2)
    tnc.test_a_sequence_with_every_key_masked(CPU)
    tnc.test_dropout_drawn_on_the_device_is_replayed_by_its_own_mask(CPU)
    if not SANITIZER_RUN:
        tnc.test_self_attention_training_without_coverage(CPU, BF16, 128, 3, 512, 8, 0.1)
        tnc.test_self_attention_training_without_coverage(CPU, F16, 33, 2, 128, 2, 0.1)
        tnc.test_encdec_attention_training_without_coverage(CPU, BF16, 40, 130, 2, 256, 2, 0.1)
        tnc.test_bias_free_encdec_function_without_coverage(CPU, F16)
    tnc.test_the_switch_keeps_the_extension_path(CPU, monkeypatch)   # sets a switch: last


@pytest.mark.parametrize("d,causal,p", [(64, True, 0.2), pytest.param(128, False, 0.2, marks=long_case),
                                        pytest.param(64, False, 0.0, marks=long_case)])
def test_batch_strided_attention_equals_packed_attention_bit_for_bit(d, causal, p):
    tnc.test_batch_strided_call_equals_packed_call_bit_for_bit(CPU, d, causal, p)


def test_split_k_epilogue_without_a_workspace_is_refused_before_any_launch(hostsim_lib):
    a = torch.randn(512, 128).to(BF16)
    b = torch.randn(512, 128).to(BF16)
    c = torch.zeros(128, 128, dtype=BF16)
    harness_lib = hostsim_lib
    harness_lib.nmtg_trace_begin()
    rc = harness_lib.hostsim_gemm_splitk_without_workspace(2, ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(b.data_ptr()),
                                                           ctypes.c_void_p(c.data_ptr()), 128, 128, 512)
    buf = ctypes.create_string_buffer(4096)
    harness_lib.nmtg_trace_end(buf, 4096)
    assert rc == -1 and b"workspace" in harness_lib.nmtg_last_error()          # NMTG_ERR_INVALID
    assert buf.value == b"" and float(c.abs().max()) == 0.0                    # nothing was launched, nothing written


# ----------------------------------------------------------------------------- decoding step
@pytest.mark.parametrize("m,n,k", [(32, 64, 8), (7, 100, 2056), (1, 256, 64)])
def test_few_row_products(monkeypatch, mi355x, m, n, k):
    monkeypatch.delenv("NMTG_GEMM_SKINNY")
    tst.test_few_row_products_match_the_tiled_kernels(CPU, BF16, m, n, k)


@pytest.mark.parametrize("dtype", HALVES)
@pytest.mark.parametrize("tk,b,e,h,masked", [(70, 2, 256, 2, True), (300, 2, 256, 8, True), (127, 2, 128, 4, False)])
def test_decode_step_kernel(mi355x, dtype, tk, b, e, h, masked):
    tst.test_decode_step_kernel_matches_the_gemm_path_and_the_oracle(CPU, dtype, tk, b, e, h, masked)


def test_incremental_decoding_with_learnable_positions(mi355x):
    trel.test_learnable_positions_step_by_step(CPU, BF16, 5)


# ----------------------------------------------------------------------------- gated / variational feed-forward, fp32 products
@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("act,rows,inner,p", [("gelu", 37, 72, 0.25), ("sigmoid", 5, 7, 0.5), ("relu", 64, 256, 0.0)])
def test_gated_activation_kernel(dtype, act, rows, inner, p):
    tff.test_gated_activation_kernel(CPU, dtype, act, rows, inner, p)


def test_gated_activation_kernel_pitched_shared_mask_and_philox():
    tff.test_gated_activation_kernel_on_a_pitched_input_with_a_mask_row_per_batch_column(CPU)
    tff.test_gated_activation_kernel_draws_the_documented_philox_stream(CPU, 9, 10)


@pytest.mark.parametrize("act,glu,residual", [("gelu", False, True), ("silu", True, False)])
def test_feed_forward_layer_variants(mi355x, act, glu, residual):
    tff.test_variational_dropout_uses_one_mask_row_per_batch_column(CPU, act, glu, residual)
    tff.test_gated_layer_in_evaluation_mode(CPU, BF16, act if glu else "sigmoid")


@pytest.mark.parametrize("act,tokens,dm,di,p", [("relu", 72, 96, 200, 0.5), ("agelu", 64, 33, 129, 0.0)])
def test_mlp_fp32(mi355x, act, tokens, dm, di, p):
    tm.test_mlp_fp32(CPU, act, tokens, dm, di, p)


@pytest.mark.parametrize("layout", ["nt", "nn", "tn"])
def test_gemm_fp32(mi355x, layout):
    tg.test_gemm_fp32_layouts_against_fp64(CPU, 130, 70, 33, layout)
    tg.test_gemm_fp32_batched_strided_views(CPU)


# ----------------------------------------------------------------------------- committed fixtures
@pytest.mark.parametrize("name", [n for n in dir(tgold) if n.startswith("test_") and n != "test_mlp_fixture"])
def test_golden_fixtures(mi355x, name):
    getattr(tgold, name)(CPU)


@pytest.mark.parametrize("act", ["gelu", "relu", "silu", "agelu"])
def test_golden_mlp_fixture(mi355x, act):
    tgold.test_mlp_fixture(CPU, act)


@pytest.mark.parametrize("name,adam_w", [("adamw", True), ("adam", False)])
def test_golden_fused_optim_fixture(name, adam_w):
    topt.test_fused_optim_golden_fixture(CPU, name, adam_w)


def test_golden_relative_attention_fixture(mi355x):
    trel.test_relative_attention_golden_fixture(CPU)


# ----------------------------------------------------------------------------- the same checks, bounds-checked
def test_every_check_again_under_address_sanitizer(hostsim_lib):
    """A child process repeats this file against an AddressSanitizer build of the same sources, with the sanitizer's
    runtime preloaded: PyTorch's host allocations then carry red zones, and any kernel load or store outside the
    tensor it was handed (a clamped index that is not clamped, a vector access across the end of a row) stops the run
    with the kernel's file and line. The child was started with the first test of this file and ran beside the others."""
    if SANITIZER_RUN:
        pytest.skip("this is the sanitizer run")
    if _sanitizer_run.get("skip"):
        pytest.skip(_sanitizer_run["skip"])
    try:
        rc = _sanitizer_run["proc"].wait(timeout=1500)
        with open(_sanitizer_run["log"]) as f:
            out = f.read()
    finally:
        if _sanitizer_run["proc"].poll() is None:
            _sanitizer_run["proc"].kill()
        os.unlink(_sanitizer_run["log"])
    assert rc == 0, out[-6000:]
