"""MI355X-native JVP flash attention (hand-written gfx950 HIP kernels behind the Python surface
of amorehead/jvp_flash_attention)."""
from .jvp_attention import MASK_CONST, MIN_SEQUENCE_LENGTH, JVPAttn, attention

__all__ = ["JVPAttn", "attention", "MASK_CONST", "MIN_SEQUENCE_LENGTH"]
__version__ = "0.1.0"
