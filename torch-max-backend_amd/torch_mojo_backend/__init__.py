"""torch_mojo_backend — the hot ATen ops of the reference package on hand-written MI355X
(gfx950) HIP kernels, behind the reference's own three surfaces:

* ``mojo_backend`` — the ``torch.compile`` backend class;
* ``MAPPING_TORCH_ATEN_TO_MOJO`` — the aten -> kernel registry (with ``map_to``);
* the eager ``mojo`` device op dispatch (``register_mojo_devices``, ``fast_aten_*``).

Public names follow torch_mojo_backend/__init__.py:11-33 of the reference.
"""

from torch_mojo_backend.mojo_device.register import register_mojo_devices
from torch_mojo_backend.mojo_device.torch_mojo_tensor import TorchMojoTensor
from torch_mojo_backend.torch_compile_backend.compiler import (
    MAPPING_TORCH_ATEN_TO_MOJO,
    MojoCompilerError,
    get_accelerators,
    mojo_backend,
)

__all__ = [
    "mojo_backend",
    "get_accelerators",
    "MAPPING_TORCH_ATEN_TO_MOJO",
    "MojoCompilerError",
    "register_mojo_devices",
    "TorchMojoTensor",
]
