"""Flash-Attention-2 for AMD MI355X behind the `jax_flash_attn2` API.

Same public names as the reference package (`jax_flash_attn2/__init__.py:15-35`);
`triton_flash_attention` is kept as an alias of the HIP operator so existing
call sites keep working.
"""

from .flash_attention import (
	AttentionConfig,
	Backend,
	FlashAttention,
	Platform,
	create_flash_attention,
)

__all__ = (
	"AttentionConfig",
	"Backend",
	"FlashAttention",
	"Platform",
	"create_flash_attention",
	"hip_flash_attention",
	"triton_flash_attention",
)

__version__ = "0.1.0"


def __getattr__(name):
	# the operator modules import torch (or jax); load them on first use only
	if name in ("hip_flash_attention", "triton_flash_attention"):
		from ._hip_op import flash_attention

		return flash_attention
	raise AttributeError(name)
