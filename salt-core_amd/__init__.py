"""MI355X-native backend for SALT's quantized decode path.

The product is the C-ABI shared library built from csrc/ (libsalt_gpu_mi355.so);
this Python package only loads it through ctypes for tests and the benchmark.
The directory name carries a hyphen, so it is imported under the module name
``salt_core_amd`` (see ``__graft_entry__.load_package``).
"""
from . import lib, synth  # noqa: F401
