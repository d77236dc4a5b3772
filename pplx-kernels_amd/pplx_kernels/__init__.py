"""MI355X-native MoE dispatch / combine with the ``pplx_kernels`` Python surface
(reference ``src/pplx_kernels/__init__.py:1-16``, minus the NVSHMEM helpers: this build has
no SHMEM layer)."""

from . import ops as ops
from .all_to_all import AllToAll as AllToAll
from .loopback import BoundStep as BoundStep
from .loopback import Graph as Graph
from .loopback import LoopbackWorld as LoopbackWorld
