"""Import path kept from the reference (kernels/flashsvdropeattn.py re-exports the prefill module)."""
from .rope_attn import *  # noqa: F401,F403
