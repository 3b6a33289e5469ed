"""Flash-Attention-2 for AMD MI355X behind the `jax_flash_attn2` API.

Same public names as the reference package (`jax_flash_attn2/__init__.py:15-35`).
`triton_flash_attention` is kept as a name of the HIP operator so existing call
sites keep working.  `jax_flash_attention` and `basic_attention_refrence` - the
reference's pure-XLA implementations, which are not GPU kernels - exist as names
that raise NotImplementedError: this package ships the HIP path only and has no
CPU or XLA fallback.
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
	"jax_flash_attention",
	"basic_attention_refrence",
)

__version__ = "0.1.0"


def hip_flash_attention(q, k, v, *args, **kwargs):
	"""The HIP operator, signature of the reference's `triton_flash_attention`
	(flash_attention_triton/_flash_attention.py:125-157).  jax arrays go through the XLA-FFI
	custom calls, torch tensors through ctypes; both reach the same C entry points.  The
	operator modules import jax / torch, so they are loaded on first use only."""
	from .flash_attention import _is_jax_array

	if _is_jax_array(q):
		from ._jax_op import flash_attention as op
	else:
		from ._hip_op import flash_attention as op
	return op(q, k, v, *args, **kwargs)


triton_flash_attention = hip_flash_attention


def jax_flash_attention(*args, **kwargs):
	"""Name of the reference's pure-XLA blockwise attention (flash_attention_jax/_flash_attention.py:32-133).
	Not part of this package."""
	raise NotImplementedError(
		"jax_flash_attention is the reference's pure-XLA implementation; this package only provides the HIP kernels "
		"(FlashAttention with Platform.HIP, or hip_flash_attention)"
	)


def basic_attention_refrence(*args, **kwargs):
	"""Name of the reference's naive fp32 attention (refrence_call.py:23-104).  Not part of this package."""
	raise NotImplementedError(
		"basic_attention_refrence is the reference's naive XLA attention; this package only provides the HIP kernels "
		"(FlashAttention with Platform.HIP, or hip_flash_attention)"
	)
