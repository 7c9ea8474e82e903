"""MI355X-native stand-in for the device work and runtime wrappers of
intel/mlir-extensions' tile pipeline: hand-written gfx950 kernels (csrc/kernels)
behind the IMEX `gpu*` runtime-wrapper C ABI (csrc/runtime), plus the
`_mlir_ciface_*` runner utilities (csrc/runner_utils).

The directory name carries a hyphen, so it is loaded by path (see
``__graft_entry__.load_package``) under the module name ``mlir_extensions_amd``.
"""
from . import build  # noqa: F401
from . import host  # noqa: F401
