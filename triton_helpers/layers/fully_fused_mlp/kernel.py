from triton_helpers_amd.layers.fully_fused_mlp import kernel as _impl

globals().update({k: v for k, v in vars(_impl).items() if not k.startswith('__')})
