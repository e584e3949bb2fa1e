from triton_helpers_amd.layers.hash_encoding.helpers import *  # noqa: F401,F403
from triton_helpers_amd.layers.hash_encoding import helpers as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith('__')})
