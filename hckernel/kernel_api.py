from hc_amd.kernel_api import *  # noqa: F401,F403
from hc_amd.kernel_api import (Buffer, CurrentGroup, CurrentGroup1, CurrentGroup2,  # noqa: F401
                               CurrentGroup3, CurrentSubGroup, CurrentWorkitem, TunableParam,
                               atomic_ref, create_mapping)
