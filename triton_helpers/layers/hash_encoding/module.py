from triton_helpers_amd.layers.hash_encoding.module import *  # noqa: F401,F403
from triton_helpers_amd.layers.hash_encoding import module as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith('__')})
