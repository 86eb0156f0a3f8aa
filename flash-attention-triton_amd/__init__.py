"""MI355X-native FlashAttention-2: same four public names as the reference package
(src/flash_attention_triton/__init__.py:13)."""

from ._configurators_v2 import BackwardConfig, KernelsConfigV2, init_to_zero_v2
from .flash_attention_2 import flash_attention_v2, flash_attention_v2_custom

__version__ = "0.1.0"
__all__ = [
    "BackwardConfig",
    "KernelsConfigV2",
    "flash_attention_v2",
    "flash_attention_v2_custom",
    "init_to_zero_v2",
]
