from hc_amd.kernel import *  # noqa: F401,F403
from hc_amd.kernel import kernel  # noqa: F401
