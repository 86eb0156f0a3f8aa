"""MI355X-native FlashAttention-2: same four public names as the reference package
(src/flash_attention_triton/__init__.py:13), plus `flash_attention_v2_op`, the same function routed
through operators registered with ``torch.library`` (traceable by ``torch.compile``)."""

from ._configurators_v2 import BackwardConfig, KernelsConfigV2, init_to_zero_v2
from .flash_attention_2 import flash_attention_v2, flash_attention_v2_custom
from ._torch_op import flash_attention_v2_op

__version__ = "0.1.0"
__all__ = [
    "BackwardConfig",
    "KernelsConfigV2",
    "flash_attention_v2",
    "flash_attention_v2_custom",
    "flash_attention_v2_op",
    "init_to_zero_v2",
]
