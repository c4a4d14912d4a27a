from kairos_amd.quant_model import *  # noqa: F401,F403
from kairos_amd import quant_model as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith("__")})
