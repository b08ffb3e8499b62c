"""ffn_kernel_amd — mask-routed linear / SwiGLU FFN for AMD MI355X (gfx950).

Drop-in for the `ffn_kernel` package of wenhaoli-xmu/ffn_kernel (ffn_kernel/__init__.py:1):
    from ffn_kernel_amd import MaskedLinear, MaskedFFN
"""
from .modules import MaskedFFNModule, MaskedLinearModule
from .ops import (MaskedFFN, MaskedLinear, Routing, masked_ffn_backward, masked_ffn_forward, masked_linear_backward,
                  masked_linear_forward, route, set_route_cache, shared_routing)

__all__ = ["MaskedLinear", "MaskedFFN", "MaskedLinearModule", "MaskedFFNModule", "masked_linear_forward",
           "masked_linear_backward", "masked_ffn_forward", "masked_ffn_backward", "Routing", "route", "shared_routing",
           "set_route_cache"]
