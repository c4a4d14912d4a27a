from kairos_amd.smooth_scale import *  # noqa: F401,F403
from kairos_amd import smooth_scale as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith("__")})
