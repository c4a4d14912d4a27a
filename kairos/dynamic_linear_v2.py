from kairos_amd.dynamic_linear_v2 import *  # noqa: F401,F403
from kairos_amd import dynamic_linear_v2 as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith("__")})
