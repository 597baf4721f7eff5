"""MI355X-native DIOPI backend for DIPU: host-side package.

  build      hipcc build of lib/libdiopi_impl.so and lib/libdipu_amd_rt.so
  diopi      ctypes view of the DIOPI C ABI (include/diopi/*.h)
  ops        op adapter mirroring torch_dipu's generated wrappers for the inference path
  runtime    device / stream / event / allocator facade (include/dipu_amd/runtime.h)
  workloads  seeded synthetic inputs for the measured configurations

The directory name contains a dot, so it is loaded by path (see __graft_entry__.load_package)
under the module name `deeplink_framework_amd`.
"""
from . import _native, diopi, ops, runtime, workloads  # noqa: F401

__all__ = ["_native", "diopi", "ops", "runtime", "workloads"]
