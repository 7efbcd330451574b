"""Builds tests/hostsim/_build/libnmtg_hostsim.so: the library's elementwise kernel sources (LayerNorm, softmax +
dropout, dropout + add, cross-entropy, the column-sum and split-K reductions) compiled as plain C++ for the CPU and run lane by lane by hostsim.cpp.

The kernel sources are used as they are, apart from three textual substitutions that C++ needs:
    extern __shared__ T name[];   ->  T* name = (T*) the simulator's dynamic-LDS block
    __shared__                    ->  static            (blocks run one after the other, so one copy is per block)
    "+v" asm register constraint  ->  "+r"              (an empty asm statement that only pins a value)
and the path of the public header. The result exports the same extern "C" entry points as libnmtg_hip.so for those
operators, plus hostsim_* hooks (stubs.cpp) for the reductions that have no entry point of their own, and takes host
pointers. Test infrastructure: python tests/hostsim/hostsim_build.py
"""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "nmtgminor_amd", "csrc")
BUILD = os.path.join(HERE, "_build")
CXX = os.environ.get("HOSTSIM_CXX", "/opt/rocm/lib/llvm/bin/clang++")
# HOSTSIM_SANITIZE=1: AddressSanitizer build (host code only). The kernels' loads and stores are then checked against
# the bounds of the tensors they are handed, when the process runs with the sanitizer's runtime preloaded:
#   HOSTSIM_SANITIZE=1 LD_PRELOAD=$(clang++ -print-file-name=libclang_rt.asan-x86_64.so) \
#   ASAN_OPTIONS=detect_leaks=0:detect_stack_use_after_return=0 python -m pytest tests/test_hostsim_cpu.py
SANITIZE = os.environ.get("HOSTSIM_SANITIZE") == "1"
# The kernel sources are compiled without optimisation: their epilogues unroll into functions of 10^5 instructions that
# take a minute each to optimise and run no faster for it (the time goes into fiber switches and the MFMA arithmetic,
# which live in hostsim.cpp and are optimised).
OPT = os.environ.get("HOSTSIM_OPT", "-O0")
LIB = os.path.join(BUILD, "libnmtg_hostsim_asan.so" if SANITIZE else "libnmtg_hostsim.so")

KERNEL_SOURCES = ["api.hip", "layer_norm.hip", "softmax_dropout.hip", "dropout_add.hip", "xentropy.hip", "reduce.hip",
                  "gemm.hip", "gemm_nt.hip", "gemm_nn.hip", "gemm_tn.hip", "mlp.hip", "attention.hip", "rel_position.hip", "multi_tensor.hip", "rotary.hip", "flash_attn.hip", "gemm_f32.hip", "glu.hip", "attn_decode.hip", "gemm_skinny.hip", "stream_probe.hip"]
HEADERS = ["common.hip.h", "trace.hip.h", "reduce.hip.h", "gemm.hip.h", "gemm_ring.hip.h", "gemm_inst.hip.h"]
OWN_SOURCES = ["hostsim.cpp", "stubs.cpp"]


# Inline assembly cannot be compiled for the host. Every statement is listed here with what it does, and a statement
# that is not listed stops the build.
ASM_REWRITES = [
    # one 1 KB global -> LDS transfer: lane l copies 16 bytes from sbase + voff to LDS address lds_addr + 16 l
    (r'asm volatile\("s_mov_b32 m0, %2\\n\\ts_nop 0\\n\\tglobal_load_lds_dwordx4 %0, %1"\s*:\s*:\s*"v"\(voff\), "s"\(sbase\), '
     r'"s"\(lds_addr\)\s*:\s*"memory", "m0"\);',
     "::hostsim::dma_issue(static_cast<const char*>(sbase) + voff, ::hostsim::lds_offset_of(lds_addr) + 16 * ::hostsim::lane_id(), 16);"),
    # LDS reads done, then the workgroup barrier
    (r'asm volatile\("s_waitcnt lgkmcnt\(0\)\\n\\ts_barrier" ::: "memory"\);', "::hostsim::sync_block();"),
]


def transform(text):
    for pattern, replacement in ASM_REWRITES:
        text = re.sub(pattern, lambda m: replacement, text)
    left = [m.group(0) for m in re.finditer(r'asm volatile\("[^"]+"', text)]
    if left:
        raise RuntimeError("hostsim: inline assembly without a host translation: %s" % left[0])
    text = re.sub(r"extern\s+__shared__\s+(?:__align__\(\d+\)\s+)?([A-Za-z_][\w:]*)\s+(\w+)\s*\[\s*\]\s*;",
                  r"\1* \2 = reinterpret_cast<\1*>(::hostsim::dynamic_lds);", text)
    text = re.sub(r"\b__shared__\b", "static", text)
    text = text.replace('"+v"', '"+r"')
    text = text.replace('"../../include/nmtg_hip.h"', '"%s"' % os.path.join(ROOT, "include", "nmtg_hip.h"))
    return text


def sources():
    out = [os.path.join(CSRC, n) for n in KERNEL_SOURCES + HEADERS if os.path.exists(os.path.join(CSRC, n))]
    out += [os.path.join(HERE, n) for n in OWN_SOURCES]
    out += [os.path.join(HERE, "shim", "hip", n) for n in os.listdir(os.path.join(HERE, "shim", "hip"))]
    out.append(os.path.abspath(__file__))
    return out


def stale():
    if not os.path.exists(LIB):
        return True
    built = os.path.getmtime(LIB)
    return any(os.path.getmtime(s) > built for s in sources())


def available():
    return os.path.exists(CXX)


def build(verbose=False):
    os.makedirs(BUILD, exist_ok=True)
    units = []
    for name in KERNEL_SOURCES + HEADERS:
        src = os.path.join(CSRC, name)
        if not os.path.exists(src):
            continue
        dst = os.path.join(BUILD, name if name.endswith(".hip.h") else name[:-len(".hip")] + ".cpp")
        with open(src) as f:
            text = '#line 1 "%s"\n' % src + transform(f.read())
        with open(dst, "w") as f:
            f.write(text)
        if not name.endswith(".hip.h"):
            units.append(dst)
    units += [os.path.join(HERE, n) for n in OWN_SOURCES]
    flags = ["-x", "c++", "-std=c++17", OPT, "-gline-tables-only", "-fPIC", "-fno-strict-aliasing", "-Wno-unknown-pragmas",
             "-Wno-pass-failed", "-Wno-unused-command-line-argument", "-I" + os.path.join(HERE, "shim"), "-I" + BUILD]
    link = []
    if SANITIZE:
        # host code only: there is no device code in this build at all (-x c++)
        flags += ["-fsanitize=address", "-fno-gpu-sanitize", "-shared-libasan", "-fno-omit-frame-pointer"]
        link = ["-fsanitize=address", "-fno-gpu-sanitize", "-shared-libasan"]
    objs = []
    procs = []
    for u in units:
        obj = os.path.join(BUILD, os.path.basename(u) + (".asan.o" if SANITIZE else ".o"))
        objs.append(obj)
        opt = ["-O2"] if os.path.dirname(u) == HERE else []
        procs.append((u, subprocess.Popen([CXX] + flags + opt + ["-c", u, "-o", obj], stdout=subprocess.PIPE,
                                          stderr=subprocess.STDOUT, text=True)))
    failed = False
    for u, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0 or verbose:
            sys.stderr.write(out)
        failed |= p.returncode != 0
    if failed:
        raise RuntimeError("hostsim: compilation failed")
    subprocess.check_call([CXX, "-shared", "-o", LIB] + link + objs)
    return LIB


def ensure():
    """Path of an up-to-date library (built on demand)."""
    if stale():
        build()
    return LIB


if __name__ == "__main__":
    if "--if-stale" in sys.argv:
        print(ensure())
    else:
        print(build(verbose=True))
