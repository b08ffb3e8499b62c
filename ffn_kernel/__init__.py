"""Import-name alias: `from ffn_kernel import MaskedLinear, MaskedFFN` (the reference's import line,
ffn_kernel/__init__.py:1, README.md:46, 81) resolves to ffn_kernel_amd's HIP-backed operators."""
from ffn_kernel_amd import *  # noqa: F401,F403
from ffn_kernel_amd import MaskedFFN, MaskedLinear, __all__  # noqa: F401
