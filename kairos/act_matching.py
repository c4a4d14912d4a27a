from kairos_amd.act_matching import *  # noqa: F401,F403
from kairos_amd import act_matching as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith("__")})
