from kairos_amd.dynamic_linear import *  # noqa: F401,F403
from kairos_amd import dynamic_linear as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith("__")})
