"""ctypes mirror of the C++ host front-end (``dali_amd/host/dali.h``).

The package is a thin scripting binding: ``Array`` handles and the ``op``
functions build the same lazy expressions a C++ user of the reference writes
(``dali/array/array.h``, ``dali/array/op.h``); planning, HIP code generation,
hipRTC compilation and launches all happen in the native libraries
``lib/libdali_front.so`` (front-end) and ``lib/libdali_hip.so`` (C ABI of
``include/dali_hip.h``). There is no CPU execution path: without the native
libraries the import fails, and without a GPU every evaluation raises.
"""
from ._native import front, hip, DaliError, lib_paths  # noqa: F401
from .array import Array, DTYPE_FLOAT, DTYPE_DOUBLE, DTYPE_INT32, eval_together, jit_stats, last_kernel_kinds, last_kernel_names, last_source, generate_only, generated_source, Recording, ScopeObserver  # noqa: F401
from . import op  # noqa: F401
