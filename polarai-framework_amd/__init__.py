"""MI355X-native device runtime for the PolarAI/Athena framework.

This package holds the Python view of the two native libraries that make up
the runtime:

* ``libpolar_hip.so``     -- the gfx950 device code behind the C ABI declared in
  ``include/polar_hip.h`` (kernels for the builtin operations, the device
  memory pool, copies, events).  ``capi`` binds it with ctypes.
* ``libpolar_rt_hip.so``  -- the C++ runtime plugin (``initContext`` /
  ``closeContext``; Device / Context / Event / allocator layer) that the
  framework's runtime driver loads, and ``libpolar_harness.so``, a small
  executor that drives the plugin the way the framework's launch lowering
  does.  ``harness`` binds the latter.

The directory name contains a hyphen, so it cannot be imported by name; load
it with ``__graft_entry__.load_package()`` (registers it as
``polarai_framework_amd``).

Nothing here falls back to a CPU implementation: if a native library is
missing, loading raises.
"""
import os

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PACKAGE_DIR)

LIB_DEVICE = os.path.join(PACKAGE_DIR, "libpolar_hip.so")
LIB_PLUGIN = os.path.join(PACKAGE_DIR, "libpolar_rt_hip.so")
LIB_HARNESS = os.path.join(PACKAGE_DIR, "libpolar_harness.so")
TOOL_LSPOLAR = os.path.join(PACKAGE_DIR, "lspolar_hip")  # lists a plugin's devices (the framework's lspolar)
