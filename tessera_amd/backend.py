"""Host-side mirror of tessera's ``Backend`` interface for the quantized-matmul path.

Names, argument meaning and error behaviour follow ``include/tessera/backend.hpp``
(``Backend`` :847-1037, ``KernelLaunch`` :45-67, ``Buffer`` :69-134) and
``include/tessera/types.hpp`` (``StatusCode`` :36-48).  Where the reference returns
``std::expected<T, StatusCode>``, these methods return ``T`` and raise
:class:`StatusError` carrying the same code.

Everything goes through the C ABI of ``libtessera_qmm.so`` (``include/tessera_qmm.h``);
there is no CPU fallback: if the library is missing or the device is not a gfx950 part,
construction or ``Init`` fails.
"""
from __future__ import annotations

import ctypes as C
import enum
import os
from dataclasses import dataclass, field
from typing import Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtessera_qmm.so")


class StatusCode(enum.IntEnum):
    Ok = 0
    InvalidArgument = 1
    FileNotFound = 2
    MalformedFile = 3
    UnsupportedFeature = 4
    OutOfMemory = 5
    DeviceError = 6
    NonFinite = 7
    NetworkError = 8


class StatusError(RuntimeError):
    """A call returned a non-Ok tessera StatusCode."""

    def __init__(self, code: int, what: str = "", detail: str = ""):
        self.code = StatusCode(code)
        msg = f"{what}: {self.code.name}" if what else self.code.name
        if detail:
            msg += f" ({detail})"
        super().__init__(msg)


def load_library(path: str = LIB_PATH) -> C.CDLL:
    """dlopen the kernel library and declare the C ABI.  Raises if it was not built."""
    if not os.path.exists(path):
        raise FileNotFoundError(
            f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C tessera_amd/csrc`")
    lib = C.CDLL(path)
    vp, sz, u64p, u32p = C.c_void_p, C.c_size_t, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)
    sig = {
        "qmm_init": (C.c_int32, [C.c_int]),
        "qmm_device_name": (C.c_char_p, []),
        "qmm_memory_info": (C.c_int32, [u64p, u64p]),
        "qmm_alloc": (C.c_int32, [sz, C.POINTER(vp)]),
        "qmm_free": (C.c_int32, [vp]),
        "qmm_copy_h2d": (C.c_int32, [vp, vp, sz, vp]),
        "qmm_copy_d2h": (C.c_int32, [vp, vp, sz, vp]),
        "qmm_copy_d2d": (C.c_int32, [vp, vp, sz, vp]),
        "qmm_load": (C.c_int32, [C.c_char_p, C.POINTER(C.c_size_t)]),
        "qmm_kernel_id": (C.c_char_p, [C.c_size_t]),
        "qmm_kernel_count": (sz, []),
        "qmm_kernel_name": (C.c_char_p, [sz]),
        "qmm_launch": (C.c_int32, [C.c_size_t, u32p, u32p, C.POINTER(vp), C.POINTER(sz), sz, u64p,
                                   sz, vp]),
        "qmm_launch_static": (C.c_int32, [C.c_size_t, u32p, u32p, C.POINTER(vp), C.POINTER(sz), sz, u64p,
                                          sz, vp]),
        "qmm_static_scratch_bytes": (sz, []),
        "qmm_workspace_bytes": (C.c_int32, [C.c_size_t, u64p, sz, C.POINTER(sz)]),
        "qmm_set_workspace": (C.c_int32, [vp, sz]),
        "qmm_set_q4k_tensor_rows": (C.c_int32, [C.c_uint32]),
        "qmm_q4k_tensor_rows": (C.c_uint32, []),
        "qmm_sync": (C.c_int32, [vp]),
        "qmm_last_error": (C.c_char_p, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


class MemoryKind(enum.IntEnum):
    Device = 0


@dataclass
class DeviceMemoryInfo:
    total_bytes: int = 0
    free_bytes: int = 0


class Buffer:
    """RAII device buffer (backend.hpp:69-134).  ``Handle()`` is the raw device address."""

    def __init__(self, backend: "Backend", handle: int, size: int, owned: bool = True):
        self._backend, self._handle, self._size, self._owned = backend, handle, size, owned

    def Handle(self) -> int:
        return self._handle

    def Size(self) -> int:
        return self._size

    def release(self) -> None:
        if self._owned and self._handle:
            self._backend.FreeBuffer(MemoryKind.Device, self._handle)
        self._handle = 0

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


class Kernel:
    """A loaded built-in (backend.hpp:1004-1020)."""

    def __init__(self, handle: int, kernel_id: str):
        self._handle, self._id = handle, kernel_id

    def Id(self) -> str:
        return self._id

    def Handle(self) -> int:
        return self._handle


@dataclass
class KernelLaunch:
    """backend.hpp:55-67: workgroup counts, workgroup size, buffers then 64-bit scalars."""

    grid_x: int = 1
    grid_y: int = 1
    grid_z: int = 1
    block_x: int = 256
    block_y: int = 1
    block_z: int = 1
    buffers: list = field(default_factory=list)
    scalars: list = field(default_factory=list)


class Backend:
    """The MI355X backend: ``Name() == "mi355x"``; one instance per process."""

    def __init__(self, lib_path: str = LIB_PATH, stream: int = 0):
        self._lib = load_library(lib_path)
        self._device_index = 0
        self._stream = C.c_void_p(stream)
        self._ready = False

    # -- identity ---------------------------------------------------------------
    def Name(self) -> str:
        return "mi355x"

    def DeviceName(self) -> str:
        return self._lib.qmm_device_name().decode()

    def MemoryInfo(self) -> DeviceMemoryInfo:
        t, f = C.c_uint64(), C.c_uint64()
        self._check(self._lib.qmm_memory_info(C.byref(t), C.byref(f)), "MemoryInfo")
        return DeviceMemoryInfo(t.value, f.value)

    def SetDeviceIndex(self, index: int) -> None:
        self._device_index = index

    def SetStream(self, stream: int) -> None:
        """Not in the reference (it owns its one stream): lets a caller that already has a HIP
        stream, e.g. torch's current stream, put the launches on it."""
        self._stream = C.c_void_p(stream)

    def Init(self) -> None:
        self._check(self._lib.qmm_init(self._device_index), "Init")
        self._ready = True

    # -- memory -----------------------------------------------------------------
    def AllocateBuffer(self, nbytes: int, kind: MemoryKind = MemoryKind.Device) -> Buffer:
        if nbytes <= 0:
            raise StatusError(StatusCode.InvalidArgument, "AllocateBuffer")
        p = C.c_void_p()
        self._check(self._lib.qmm_alloc(nbytes, C.byref(p)), "AllocateBuffer")
        return Buffer(self, p.value, nbytes)

    def WrapBuffer(self, handle: int, nbytes: int) -> Buffer:
        """A Buffer over memory somebody else owns (a torch tensor's ``data_ptr()``)."""
        return Buffer(self, handle, nbytes, owned=False)

    def FreeBuffer(self, kind: MemoryKind, handle: int) -> None:
        self._lib.qmm_free(C.c_void_p(handle))

    def CopyH2D(self, dst: Buffer, src) -> None:
        self.CopyH2DAt(dst, 0, src)

    def CopyH2DAt(self, dst: Buffer, offset: int, src) -> None:
        host = np.ascontiguousarray(src)
        if offset < 0 or offset + host.nbytes > dst.Size():
            raise StatusError(StatusCode.InvalidArgument, "CopyH2DAt")
        self._check(self._lib.qmm_copy_h2d(C.c_void_p(dst.Handle() + offset), host.ctypes.data,
                                           host.nbytes, self._stream), "CopyH2DAt")

    def CopyD2H(self, src: Buffer, nbytes: int | None = None, dtype=np.uint8) -> np.ndarray:
        return self.CopyD2HAt(src, 0, src.Size() if nbytes is None else nbytes, dtype)

    def CopyD2HAt(self, src: Buffer, offset: int, nbytes: int, dtype=np.uint8) -> np.ndarray:
        if offset < 0 or nbytes < 0 or offset + nbytes > src.Size():
            raise StatusError(StatusCode.InvalidArgument, "CopyD2HAt")
        host = np.empty(nbytes, dtype=np.uint8)
        self._check(self._lib.qmm_copy_d2h(host.ctypes.data, C.c_void_p(src.Handle() + offset),
                                           nbytes, self._stream), "CopyD2HAt")
        return host.view(dtype)

    def CopyD2D(self, dst: Buffer, dst_offset: int, src: Buffer, src_offset: int, nbytes: int) -> None:
        if (dst_offset < 0 or src_offset < 0 or nbytes < 0 or dst_offset + nbytes > dst.Size()
                or src_offset + nbytes > src.Size()):
            raise StatusError(StatusCode.InvalidArgument, "CopyD2D")
        self._check(self._lib.qmm_copy_d2d(C.c_void_p(dst.Handle() + dst_offset),
                                           C.c_void_p(src.Handle() + src_offset), nbytes,
                                           self._stream), "CopyD2D")

    # -- kernels ----------------------------------------------------------------
    def LoadKernel(self, name: str, code: bytes = b"") -> Kernel:
        if code:
            # Built-ins only, as on the reference ROCm backend (rocm_backend.cpp:639-670).
            raise StatusError(StatusCode.UnsupportedFeature, "LoadKernel")
        h = C.c_size_t()
        self._check(self._lib.qmm_load(name.encode(), C.byref(h)), f"LoadKernel({name})")
        return Kernel(h.value, name)

    def FreeKernel(self, handle: int) -> None:  # handles are table indices; nothing to free
        return None

    def KernelNames(self) -> list[str]:
        return [self._lib.qmm_kernel_name(i).decode() for i in range(self._lib.qmm_kernel_count())]

    def LaunchKernel(self, kernel: Kernel, launch: KernelLaunch, no_alloc: bool = False) -> None:
        """``no_alloc=True`` goes through ``qmm_launch_static`` (not in the reference): the same
        launch with every kernel's scratch taken from the library's static device array, for
        callers that may not allocate device memory."""
        nb, ns = len(launch.buffers), len(launch.scalars)
        grid = (C.c_uint32 * 3)(launch.grid_x, launch.grid_y, launch.grid_z)
        block = (C.c_uint32 * 3)(launch.block_x, launch.block_y, launch.block_z)
        bufs = (C.c_void_p * max(nb, 1))(*[b.Handle() for b in launch.buffers])
        sizes = (C.c_size_t * max(nb, 1))(*[b.Size() for b in launch.buffers])
        scal = (C.c_uint64 * max(ns, 1))(*[int(s) & 0xFFFFFFFFFFFFFFFF for s in launch.scalars])
        entry = self._lib.qmm_launch_static if no_alloc else self._lib.qmm_launch
        self._check(entry(kernel.Handle(), grid, block, bufs, sizes, nb, scal, ns, self._stream),
                    f"LaunchKernel({kernel.Id()})")

    def WorkspaceBytes(self, kernel: Kernel, scalars: Sequence[int]) -> int:
        """Scratch a launch of ``kernel`` with these scalars needs (``qmm_workspace_bytes``)."""
        ns = len(scalars)
        scal = (C.c_uint64 * max(ns, 1))(*[int(s) & 0xFFFFFFFFFFFFFFFF for s in scalars])
        out = C.c_size_t()
        self._check(self._lib.qmm_workspace_bytes(kernel.Handle(), scal, ns, C.byref(out)), "WorkspaceBytes")
        return int(out.value)

    def SetWorkspace(self, buffer: "Buffer | None") -> None:
        """Hand the library a caller-owned workspace (``qmm_set_workspace``); ``None`` clears it.
        Mirrors the scratch the reference's arch state owns (project.cpp:127-155)."""
        if buffer is None:
            self._check(self._lib.qmm_set_workspace(None, 0), "SetWorkspace")
        else:
            self._check(self._lib.qmm_set_workspace(C.c_void_p(buffer.Handle()), buffer.Size()), "SetWorkspace")

    def SetQ4KTensorRows(self, rows: int) -> None:
        """Row count from which the Q4_K ids other than gemm_q4k_wmma use the fp16 tensor-core tile
        (``qmm_set_q4k_tensor_rows``; default 64 as the reference's table, at least 17, 0 = default)."""
        self._check(self._lib.qmm_set_q4k_tensor_rows(int(rows)), "SetQ4KTensorRows")

    def Q4KTensorRows(self) -> int:
        return int(self._lib.qmm_q4k_tensor_rows())

    def StaticScratchBytes(self) -> int:
        return int(self._lib.qmm_static_scratch_bytes())

    def Synchronize(self) -> None:
        self._check(self._lib.qmm_sync(self._stream), "Synchronize")

    # -- helpers ----------------------------------------------------------------
    def Upload(self, host) -> Buffer:
        """AllocateBuffer + CopyH2D of a numpy array."""
        host = np.ascontiguousarray(host)
        buf = self.AllocateBuffer(max(host.nbytes, 1))
        if host.nbytes:
            self.CopyH2D(buf, host)
        return buf

    def _check(self, code: int, what: str) -> None:
        if code != 0:
            raise StatusError(code, what, self._lib.qmm_last_error().decode(errors="replace"))


_BACKEND: Backend | None = None


def CreateBackend() -> Backend:
    """tessera::CreateBackend() (backend.hpp:1062-1064): the process-wide backend, initialised."""
    global _BACKEND
    if _BACKEND is None:
        b = Backend()
        b.Init()
        _BACKEND = b
    return _BACKEND


def launch(backend: Backend, kernel: Kernel, buffers: Sequence[Buffer], scalars: Sequence[int],
           grid=(1, 1, 1), block=(256, 1, 1)) -> None:
    backend.LaunchKernel(kernel, KernelLaunch(grid[0], grid[1], grid[2], block[0], block[1],
                                              block[2], list(buffers), list(scalars)))
