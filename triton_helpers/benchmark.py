from triton_helpers_amd.benchmark import *  # noqa: F401,F403
from triton_helpers_amd import benchmark as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith('__')})
