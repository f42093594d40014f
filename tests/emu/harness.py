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


class _Host(torch.Tensor):
    """What torch.from_numpy returns here: a CPU tensor over the array whose .cuda() copies it into
    the model's device memory."""

    def cuda(self):
        plain = self.as_subclass(torch.Tensor)
        t = self._emu_device.empty(tuple(plain.shape), dtype=plain.dtype)
        t.copy_(plain)
        return t


class _Stream:
    """Every stream is the one synchronous stream of the model."""
    cuda_stream = 0

    def wait_stream(self, other):
        pass

    def synchronize(self):
        pass


class _Graph:
    def __init__(self, library):
        self._lib, self._h = library, None

    def replay(self):
        assert self._h, "a graph that was never captured"
        assert self._lib.emu_graph_launch(self._h) == 0, "a launch of the graph failed"

    def __del__(self):
        if self._h:
            self._lib.emu_graph_destroy(self._h)


class _Capture:
    def __init__(self, library, graph):
        self._lib, self._graph = library, graph

    def __enter__(self):
        self._lib.emu_graph_begin_capture()
        return self

    def __exit__(self, *exc):
        self._graph._h = self._lib.emu_graph_end_capture()
        return False


class _Nothing:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


class _Cuda:
    """torch.cuda, as far as the tests use it: streams (all the one synchronous stream), graphs
    (the model's record-and-replay of launches), the free-memory query (from the model's list of
    allocations)."""
    TOTAL = 288 << 30

    def __init__(self, library):
        self._lib = library
        for name in ("emu_graph_begin_capture", "emu_graph_end_capture"):
            getattr(library, name).restype = C.c_void_p
        library.emu_graph_launch.argtypes = [C.c_void_p]
        library.emu_graph_destroy.argtypes = [C.c_void_p]
        library.emu_live_bytes.restype = C.c_size_t

    def synchronize(self):
        pass

    def empty_cache(self):
        pass

    def Stream(self):
        return _Stream()

    def current_stream(self):
        return _Stream()

    def stream(self, s):
        return _Nothing()

    def CUDAGraph(self):
        return _Graph(self._lib)

    def graph(self, graph, stream=None):
        return _Capture(self._lib, graph)

    def mem_get_info(self):
        return self.TOTAL - int(self._lib.emu_live_bytes()), self.TOTAL

    def memory_reserved(self):
        return int(self._lib.emu_live_bytes())

    memory_allocated = memory_reserved


class EmuTorch:
    """`torch`, for code that allocates "cuda" tensors and synchronises: the tensors are CPU
    tensors over the model's device memory."""
    uint8, int32, int64, float32 = torch.uint8, torch.int32, torch.int64, torch.float32
    equal = staticmethod(torch.equal)

    def __init__(self, library):
        self._lib = library
        self._lib.emu_alloc_buffer.restype = C.c_void_p
        self._lib.emu_alloc_buffer.argtypes = [C.c_size_t, C.c_size_t]
        self._lib.emu_free_buffer.argtypes = [C.c_void_p]
        self._live = []
        self.cuda = _Cuda(library)

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
        host = torch.from_numpy(np.ascontiguousarray(array)).as_subclass(_Host)
        host._emu_device = self
        return host

    def release(self):
        """Frees every buffer handed out (tensors over them must not be touched afterwards)."""
        for ptr in self._live:
            self._lib.emu_free_buffer(ptr)
        self._live = []
