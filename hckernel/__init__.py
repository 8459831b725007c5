"""Import-compatible face of hc_amd: `from hckernel.kernel import *` resolves to
the MI355X-native implementation, so kernels written against the reference's
package name run unchanged (python/hckernel/tests/test_e2e.py:6)."""
