"""Python side of the library-level CPU tests (TEST INFRASTRUCTURE): the product's own ctypes
binding bound to libhomcomp_emu.so (the library's source built for the host against the execution
model, gen_sources.build_library), and a stand-in for the few torch calls that the GPU tests'
helper (tests/gpu_util.Gpu) makes, backed by the model's "device memory".

Why the buffers must come from here: a workgroup is a process, so what a kernel writes is only
seen by the caller in shared memory, and every access a kernel makes is checked against the list
of allocations (each ends at an inaccessible page)."""
from __future__ import annotations

import ctypes as C
import importlib.util
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def _load(name, path):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def load_binding(library_path: str):
    """A second instance of the package's binding module, bound to `library_path`."""
    mod = _load("homcomp_binding_on_the_cpu_model", os.path.join(ROOT, "tirocinio-triennale_amd", "__init__.py"))
    mod.LIB_PATH = library_path
    mod._stream_ptr = lambda stream: 0          # every stream is the synchronous one here
    return mod


class _Host:
    """What torch.from_numpy returns, as far as the helpers go: something with .cuda()."""

    def __init__(self, dev, array):
        self._dev, self._array = dev, np.ascontiguousarray(array)

    def cuda(self):
        t = self._dev.empty(self._array.shape, dtype=torch.from_numpy(self._array).dtype)
        t.copy_(torch.from_numpy(self._array))
        return t


class EmuTorch:
    """`torch`, for code that allocates "cuda" tensors and synchronises: the tensors are CPU
    tensors over the model's device memory."""
    uint8, int32, int64, float32 = torch.uint8, torch.int32, torch.int64, torch.float32
    equal = staticmethod(torch.equal)

    class cuda:
        synchronize = staticmethod(lambda: None)

    def __init__(self, library):
        self._lib = library
        self._lib.emu_alloc_buffer.restype = C.c_void_p
        self._lib.emu_alloc_buffer.argtypes = [C.c_size_t, C.c_size_t]
        self._lib.emu_free_buffer.argtypes = [C.c_void_p]
        self._live = []

    def empty(self, shape, dtype=torch.float32, device="cuda"):
        assert device == "cuda"
        count = int(np.prod(shape)) if not isinstance(shape, int) else shape
        item = torch.empty(0, dtype=dtype).element_size()
        nbytes = max(count * item, 1)
        # byte buffers end at their last byte (an access one byte too far is a fault); arrays of
        # numbers start at a multiple of 16, as the library asks of its operands
        ptr = self._lib.emu_alloc_buffer(nbytes, 1 if item == 1 else 16)
        if not ptr:
            raise MemoryError("the model's device memory")
        self._live.append(ptr)
        raw = np.ctypeslib.as_array((C.c_uint8 * nbytes).from_address(ptr))
        return torch.from_numpy(raw)[:count * item].view(dtype).reshape(shape if not isinstance(shape, int) else (shape,))

    def zeros(self, shape, dtype=torch.float32, device="cuda"):
        t = self.empty(shape, dtype, device)
        t.zero_()
        return t

    def full(self, shape, value, dtype=torch.float32, device="cuda"):
        t = self.empty(shape, dtype, device)
        t.fill_(value)
        return t

    def from_numpy(self, array):
        return _Host(self, array)

    def release(self):
        """Frees every buffer handed out (tensors over them must not be touched afterwards)."""
        for ptr in self._live:
            self._lib.emu_free_buffer(ptr)
        self._live = []
