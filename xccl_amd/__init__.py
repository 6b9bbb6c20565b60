"""xccl_amd -- MI355X-native memory component for XCCL's GPU reduction path.

The product is three shared objects under ``xccl_amd/lib`` built from
``xccl_amd/csrc`` (see ``xccl_amd.build``):

* ``xccl_rocm_mem_component.so`` -- the plugin libxccl dlopens; C host side on
  the HIP runtime plus hand-written gfx950 kernels;
* ``libxccl_mc.so`` -- XCCL's mem-component dispatcher, standalone;
* ``libxccl_rocm_benchkit.so`` -- synthetic-input kernels for bench and tests.

The Python modules are thin ctypes bindings over their C ABI (``include/*.h``):
``xccl_amd.mc`` mirrors the dispatcher's functions one to one, ``xccl_amd.hip``
binds the handful of HIP runtime calls tests and bench need for device memory,
copies and events.  There is no CPU implementation of the arithmetic in this
package: without the built libraries every entry point raises.
"""
from .types import Dt, Op, Status, MemType, StreamType, dt_size  # noqa: F401

__all__ = ["Dt", "Op", "Status", "MemType", "StreamType", "dt_size"]
