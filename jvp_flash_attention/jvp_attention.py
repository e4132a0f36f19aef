"""Drop-in import path of the reference (``jvp_flash_attention.jvp_attention``)."""
from jvp_flash_attention_amd.jvp_attention import (  # noqa: F401
    MASK_CONST,
    MIN_SEQUENCE_LENGTH,
    JVPAttn,
    attention,
    is_blackwell,
    is_cuda,
    is_hip,
    supports_host_descriptor,
    supports_tma,
)
