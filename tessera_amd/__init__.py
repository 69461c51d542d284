"""MI355X (gfx950) implementation of tessera's quantized-matmul path.

``tessera_amd.backend`` mirrors the reference ``Backend`` interface over the C ABI of
``libtessera_qmm.so``; ``tessera_amd.synth`` generates seeded tensors in the reference's
weight-buffer layouts; ``tessera_amd/csrc`` holds the HIP kernels and the C ABI.
"""
from .backend import (Backend, Buffer, CreateBackend, Kernel, KernelLaunch, MemoryKind,  # noqa: F401
                      StatusCode, StatusError, launch, load_library)
