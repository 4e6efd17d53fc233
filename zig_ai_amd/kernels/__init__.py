"""Python side of the HIP kernels: ``build`` compiles and loads ``csrc/*.hip``,
``ops`` checks arguments and launches."""

from . import build, ops  # noqa: F401
from .ops import KernelError  # noqa: F401
from .build import KernelBuildError  # noqa: F401
