from kairos_amd.perf_profiler_v2 import *  # noqa: F401,F403
from kairos_amd import perf_profiler_v2 as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith("__")})
