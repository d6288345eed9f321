"""The Python package on the host model: comp_inference_amd's operators and modules called with CPU tensors, the
library underneath being tests/hostmodel/libci_hostmodel.so instead of the GPU build.  For tests of the host logic
above the C ABI (module compression, the runtime modules and their caches, package save / load) without a GPU.  The
product itself has no such mode: everything here is patched in from outside, for the duration of a `with` block, in
a process of the test's own."""
from __future__ import annotations

import contextlib
import os
import ctypes as C

import torch


class _Stream:
    cuda_stream = 0


class _Event:
    """torch.cuda.Event for code that times a launch: no time passes on the model."""

    def __init__(self, *a, **k):
        pass

    def record(self, *a, **k):
        pass

    def synchronize(self):
        pass

    def elapsed_time(self, other):
        return 1e-3


class _Properties:
    """torch.cuda.get_device_properties for code that asks for the CU count."""

    name, gcnArchName, total_memory = "host model", "gfx950:host-model", 288 << 30

    def __init__(self, cus):
        self.multi_processor_count = cus


_CPU = torch.device("cpu")


def _is_cuda(v) -> bool:
    return (isinstance(v, torch.device) and v.type == "cuda") or (isinstance(v, str) and v.startswith("cuda"))


def _moved(t: torch.Tensor) -> torch.Tensor:
    """What arrives on a GPU is a fresh, aligned allocation; a tensor that already is one stays itself (as a tensor
    that is on the GPU already does), a view at an odd offset -- tensors read from one file buffer -- is copied."""
    if t.numel() and (t.data_ptr() % 64 or not t.is_contiguous()):
        return t.clone(memory_format=torch.contiguous_format)
    return t


class _CudaMeansCpu(torch.overrides.TorchFunctionMode):
    """Inside this mode a tensor asked to go to "cuda" stays on the CPU: `.cuda()` returns the tensor, and a device
    argument that names a GPU is replaced by the CPU.  So code (and tests) written for the GPU run unchanged on the
    host model."""

    def __torch_function__(self, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        if func is torch.Tensor.cuda:
            return _moved(args[0])
        if func is torch.device:
            return func("cpu") if args and _is_cuda(args[0]) else func(*args, **kwargs)
        cpu = _CPU
        # (`.to(device)`: in the package the device is the input's, i.e. a CPU device here, where on the GPU it is a
        # real host-to-device copy whenever the tensor came from a file)
        moving = func is torch.Tensor.to and any(isinstance(a, torch.device) or _is_cuda(a) for a in list(args) + list(kwargs.values()))
        args = tuple(cpu if _is_cuda(a) else a for a in args)
        kwargs = {k: (cpu if _is_cuda(v) else v) for k, v in kwargs.items()}
        if kwargs.get("pin_memory"):
            kwargs["pin_memory"] = False  # (page-locked memory is the GPU runtime's to give)
        if func is torch.Tensor.pin_memory:
            return args[0]
        out = func(*args, **kwargs)
        return _moved(out) if moving else out


@contextlib.contextmanager
def python_api_on_hostmodel(cus: int = 8):
    from unittest import mock

    from comp_inference_amd import _lib, ccore
    from tests.hostmodel import build

    path = os.environ.get("CI_HOSTMODEL_LIB") or build.build()  # (a build with a deliberate mistake: see Model)
    saved = (_lib._lib, _lib.LIB_PATH)
    _lib._lib, _lib.LIB_PATH = None, path
    lib = _lib.lib()  # the product's own loader sets the return types
    lib.sim_init()
    lib.sim_set_cus(cus)
    lib.sim_trust_foreign_memory(1)  # the tensors are torch's: the page guards and exact extents do not apply to them
    lib.sim_violation.restype = C.c_char_p
    cpu = torch.device("cpu")
    patches = [
        mock.patch.object(_lib, "require_device", lambda t: None),
        mock.patch.object(_lib, "stream_handle", lambda device: C.c_void_p(0)),
        mock.patch.object(ccore, "_dev", lambda: cpu),
        mock.patch.object(torch.cuda, "device", lambda d: contextlib.nullcontext()),
        mock.patch.object(torch.cuda, "current_stream", lambda d=None: _Stream()),
        mock.patch.object(torch.cuda, "current_device", lambda: 0),
        mock.patch.object(torch.cuda, "set_device", lambda d: None),
        mock.patch.object(torch.cuda, "synchronize", lambda device=None: None),
        mock.patch.object(torch.cuda, "Event", _Event),
        mock.patch.object(torch.cuda, "memory_allocated", lambda device=None: 0),
        mock.patch.object(torch.cuda, "is_available", lambda: True),
        mock.patch.object(torch.cuda, "get_device_properties", lambda d=None: _Properties(cus)),
        mock.patch.object(torch.cuda, "empty_cache", lambda: None),
        # operands are "on the GPU" wherever the package asks (the host model is the GPU here)
        mock.patch.object(torch.Tensor, "is_cuda", property(lambda self: True)),
    ]
    # tests written for the GPU move things there with .cuda() / .to("cuda"): here everything stays where it is
    patches.append(_CudaMeansCpu())
    # modules that imported the helpers by name hold their own references
    import comp_inference_amd as pkg
    for name in ("linear_hip", "transposed_linear_hip", "embedding_hip", "rans_hip", "ccore", "comp_inference", "pytorch_runtime"):
        mod = getattr(pkg, name, None)
        if mod is None:
            continue
        for attr, repl in (("require_device", lambda t: None), ("stream_handle", lambda device: C.c_void_p(0))):
            if hasattr(mod, attr):
                patches.append(mock.patch.object(mod, attr, repl))
    try:
        with contextlib.ExitStack() as stack:
            for p in patches:
                stack.enter_context(p)
            yield lib
            n = lib.sim_violation_count()
            assert n == 0, [lib.sim_violation(i).decode() for i in range(n)]
    finally:
        lib.sim_trust_foreign_memory(0)
        _lib._lib, _lib.LIB_PATH = saved
