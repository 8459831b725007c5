from hc_amd.typename import Typename, typename  # noqa: F401
