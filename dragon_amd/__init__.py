"""MI355X-native LayerNorm / GroupNorm / BatchNorm / Softmax kernels behind
Dragon's ``kernels::`` interface.

``dragon_amd.kernels`` mirrors the reference's ``kernels::`` / ``math::`` free
functions over device tensors; every call goes through the C ABI of
``include/dragon_hip.h`` into hand-written gfx950 kernels. There is no CPU
fallback: importing ``dragon_amd.kernels`` without the built library raises.
"""

__version__ = "0.1.0"
