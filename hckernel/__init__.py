"""Import-compatible face of hc_amd: `from hckernel.kernel import *` resolves to
the MI355X-native implementation, so kernels written against the reference's
package name run unchanged (python/hckernel/tests/test_e2e.py:6).

This directory defines the two modules this build replaces: `hckernel.kernel`
(the GPU decorator and, through it, every name a kernel body uses) and
`hckernel.py_runtime` (the ctypes face of the runtime library).  Everything
else of the reference's package (`hckernel.kernel_sim`, its NumPy simulator,
python/hckernel/kernel_sim.py:177-203, with the `kernel_api`, `indexing` and
`typename` modules it imports relatively) resolves to the next `hckernel`
directory on the module search path: the package path is extended over all of
them, so with this repository in front of a checkout of the reference
`from hckernel.kernel_sim import kernel` still finds the reference's simulator,
complete."""
from pkgutil import extend_path

__path__ = extend_path(__path__, __name__)
