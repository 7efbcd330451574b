"""Routes the Python stand-ins to the CPU build of the kernels (tests/hostsim) — TEST INFRASTRUCTURE ONLY.

`install(setter)` points nmtgminor_amd._lib at libnmtg_hostsim.so and removes what ties the stand-ins to a GPU:
the device check, the HIP stream, the Philox (seed, offset) taken from PyTorch's device generator. It also makes the
host behave like device memory where the tests rely on it: `tensor.to(device)` returns a copy (the in-place operators
would otherwise change the inputs the oracle is given afterwards) and byte workspaces are 256-byte aligned, as device
allocations are. `setter(obj, name, value)` is pytest's monkeypatch.setattr, or plain setattr for a script.
"""
import ctypes
import importlib
import os
import pkgutil
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import hostsim_build  # noqa: E402

from nmtgminor_amd import _lib  # noqa: E402

_loaded = {}


def library():
    path = hostsim_build.ensure()
    if path not in _loaded:
        lib = ctypes.CDLL(path)
        lib.nmtg_last_error.restype = ctypes.c_char_p
        lib.nmtg_version.restype = ctypes.c_int
        for name in _lib.header_functions():
            if hasattr(lib, name) and (name.endswith("_parts") or name.endswith("_bytes")):
                getattr(lib, name).restype = ctypes.c_int64
        _loaded[path] = lib
    return _loaded[path]


def install(setter, fake_gpu=False):
    """fake_gpu: also answer torch.cuda.is_available() with True and map device='cuda' to the host, so that whole GPU
    test files can be run unchanged (tests/hostsim/rehearse.py)."""
    lib = library()
    setter(_lib, "_lib", lib)                                        # what _lib.load() hands out
    setter(_lib, "require_cuda", lambda *t: None)
    setter(_lib, "stream_of", lambda t: ctypes.c_void_p(0))

    # one Philox stream: the offset advances by 4 per draw, a manual seed restarts it (as the device generator does)
    state = {"seed": 1234, "draws": 0}

    def seed_offset(dev, n):
        state["draws"] += 1
        return state["seed"], 4 * (state["draws"] - 1)

    def manual_seed(seed):
        state["seed"], state["draws"] = int(seed), 0

    import nmtgminor_amd.native
    for m in pkgutil.walk_packages(nmtgminor_amd.native.__path__, "nmtgminor_amd.native."):
        importlib.import_module(m.name)
    for name, mod in list(sys.modules.items()):
        if name.startswith("nmtgminor_amd") and hasattr(mod, "philox_seed_offset"):
            setter(mod, "philox_seed_offset", seed_offset)
    setter(torch.cuda, "manual_seed", manual_seed)

    cpu = torch.device("cpu")
    plain_to = torch.Tensor.to

    def copying_to(self, *a, **k):
        a = list(a)
        device_given = False
        for i, x in enumerate(a):
            if isinstance(x, torch.device):
                device_given = True
                if fake_gpu and x.type == "cuda":
                    a[i] = cpu
        if isinstance(k.get("device"), torch.device):
            device_given = True
            if fake_gpu and k["device"].type == "cuda":
                k["device"] = cpu
        out = plain_to(self, *a, **k)
        if device_given and out.numel() > 0 and out.data_ptr() == self.data_ptr():
            out = out.clone()
        return out
    setter(torch.Tensor, "to", copying_to)

    plain_empty = torch.empty

    def host_device(k):
        d = k.get("device")
        if fake_gpu and ((isinstance(d, torch.device) and d.type == "cuda") or (isinstance(d, str) and d.startswith("cuda"))):
            k["device"] = cpu

    def aligned_empty(*a, **k):
        host_device(k)
        if k.get("dtype") == torch.uint8 and len(a) == 1 and isinstance(a[0], int):
            buf = plain_empty(a[0] + 256, **k)
            off = (-buf.data_ptr()) % 256
            return buf[off:off + a[0]]
        return plain_empty(*a, **k)
    setter(torch, "empty", aligned_empty)

    if fake_gpu:
        setter(torch.cuda, "is_available", lambda: True)
        setter(torch.cuda, "synchronize", lambda *a, **k: None)

        class Generator:
            def initial_seed(self):
                return state["seed"]
        setter(torch.cuda, "default_generators", (Generator(),))
        for fname in ("randn", "zeros", "ones", "rand", "randint", "full", "tensor", "arange"):
            def wrapped(*a, _f=getattr(torch, fname), **k):
                host_device(k)
                return _f(*a, **k)
            setter(torch, fname, wrapped)
    return lib
