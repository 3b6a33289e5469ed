"""Public facade: configuration, validation and platform dispatch.

Mirrors `jax_flash_attn2/flash_attention.py` of the reference name for name
(`Backend` :74-79, `Platform` :82-87, `AttentionConfig` :90-114,
`FlashAttention` :117-356, `create_flash_attention` :359-381) and adds one
platform, `Platform.HIP`, which is the default on a GPU backend and the only
one this package implements: hand-written gfx950 kernels behind the C ABI of
libfa2_hip.so.  `Platform.TRITON` and `Platform.PALLAS` on a GPU resolve to the
HIP platform (the reference likewise redirects Pallas-on-GPU to its GPU kernel,
:274-289); there is no second code path.
"""

from __future__ import annotations

import typing as tp
import warnings
from dataclasses import dataclass
from enum import Enum

AVAILABLE_FLASH_ATTENTION2_PLATFORMS = tp.Literal["triton", "pallas", "jax", "hip"]
AVAILABLE_BACKENDS = tp.Literal["gpu", "tpu", "cpu"]


class Backend(str, Enum):
	"""Device family the arrays live on (values as in the reference, :74-79)."""

	GPU = "gpu"
	TPU = "tpu"
	CPU = "cpu"


class Platform(str, Enum):
	"""Kernel family; `HIP` is the one this package implements (others: :82-87)."""

	TRITON = "triton"
	PALLAS = "pallas"
	JAX = "jax"
	HIP = "hip"


def _detect_backend() -> str:
	"""The reference asks jax (`get_backend().platform`, :102).  Without jax the
	presence of a ROCm device decides."""
	try:
		from jax.extend.backend import get_backend  # type: ignore

		plat = get_backend().platform
		return "gpu" if plat in ("gpu", "rocm", "cuda") else plat
	except Exception:
		pass
	try:
		import torch

		return "gpu" if torch.cuda.is_available() else "cpu"
	except Exception:
		return "cpu"


@dataclass
class AttentionConfig:
	"""Field for field the reference's dataclass (:90-99).  The block sizes are kept
	for source compatibility; the gfx950 kernels use fixed, measured tile shapes."""

	blocksize_q: int = 128
	blocksize_k: int = 128
	softmax_scale: tp.Optional[float] = None
	backend: tp.Optional[Backend] = None
	platform: tp.Optional[Platform] = None

	def __post_init__(self):
		if self.backend is None:
			self.backend = Backend(_detect_backend())

		if self.platform is None:
			self.platform = self._default_platform()

	def _default_platform(self) -> Platform:
		return _DEFAULT_PLATFORM.get(self.backend)


_DEFAULT_PLATFORM = {Backend.GPU: Platform.HIP, Backend.CPU: Platform.JAX, Backend.TPU: Platform.PALLAS}

# (backend, platform) pairs the constructor accepts: the reference's list (:124-132) plus HIP on a GPU
_ACCEPTED_PAIRS = frozenset(
	[(Backend.GPU, pl) for pl in (Platform.HIP, Platform.TRITON, Platform.PALLAS, Platform.JAX)]
	+ [(Backend.CPU, Platform.JAX), (Backend.TPU, Platform.JAX), (Backend.TPU, Platform.PALLAS)]
)


def _is_jax_array(x) -> bool:
	return type(x).__module__.split(".")[0] in ("jax", "jaxlib")


class FlashAttention:
	"""The reference's operator object (:117-356): validates the configuration once,
	then dispatches every call to the platform's kernels."""

	def __init__(self, config: tp.Optional[AttentionConfig] = None):
		self.config = config or AttentionConfig()
		self._validate_config()

	def _validate_config(self):
		pair = (self.config.backend, self.config.platform)
		if pair not in _ACCEPTED_PAIRS:
			raise ValueError(f"Invalid backend-platform combination: {pair[0]}-{pair[1]}")

	@staticmethod
	def repeat_kv_heads(key, value, num_reps: int):
		"""Repeats key and value heads to match query heads ("b s h d -> b s (h r) d").
		The HIP platform never calls this: its kernels read kv-head h // r directly."""
		import einops

		return (
			einops.repeat(key, "b s h d -> b s (h r) d", r=num_reps),
			einops.repeat(value, "b s h d -> b s (h r) d", r=num_reps),
		)

	def _handle_bias(self, bias, num_q_heads: int, num_kv_heads: int):
		"""Processes attention bias based on head configuration.  A bias with one
		entry per KV head is accepted as is (the reference repeats it to the query
		heads, :161-164; the HIP kernels index it by h // r instead)."""
		if bias is None or bias.shape[1] in (num_q_heads, 1, num_kv_heads):
			return bias
		raise ValueError(
			f"Incompatible bias shape. Got {bias.shape[1]} heads, expected {num_q_heads}, {num_kv_heads}, or 1"
		)

	def __call__(
		self,
		query,
		key,
		value,
		bias=None,
		attention_mask=None,
		dropout_prob: float = 0.0,
		causal: bool = False,
		dropout_seed: tp.Optional[int] = None,
		adjust_sharindgs: bool = False,
	):
		"""query [B, Sq, Hq, D], key/value [B, Sk, Hkv, D] -> [B, Sq, Hq, D]
		(signature and checks of the reference's `__call__`, :171-214)."""
		num_q_heads, num_kv_heads = query.shape[2], key.shape[2]
		if num_q_heads % num_kv_heads != 0:
			raise ValueError(
				f"Query heads ({num_q_heads}) must be divisible by key/value heads ({num_kv_heads})"
			)
		bias = self._handle_bias(bias, num_q_heads, num_kv_heads)
		kw = dict(
			query=query,
			key=key,
			value=value,
			bias=bias,
			adjust_sharindgs=adjust_sharindgs,
			attention_mask=attention_mask,
			causal=causal,
			dropout_prob=dropout_prob,
			dropout_seed=dropout_seed,
		)
		if self.config.platform == Platform.HIP:
			return self._compute_hip(**kw)
		elif self.config.platform in (Platform.TRITON, Platform.PALLAS):
			if self.config.backend != Backend.GPU:
				raise NotImplementedError(
					f"platform {self.config.platform.value!r} on backend {self.config.backend.value!r} "
					"is not part of this package (HIP kernels for AMD GPUs only)"
				)
			warnings.warn(
				f"{self.config.platform.value}-FlashAttention is not built for AMD GPUs (hip platform will be used)",
				stacklevel=1,
			)
			return self._compute_hip(**kw)
		else:  # Platform.JAX
			raise NotImplementedError(
				"Platform.JAX is the reference's pure-XLA implementation; this package only provides Platform.HIP"
			)

	forward = __call__

	def _compute_hip(
		self,
		query,
		key,
		value,
		bias=None,
		attention_mask=None,
		dropout_prob: float = 0.0,
		causal: bool = False,
		dropout_seed: tp.Optional[int] = None,
		adjust_sharindgs: bool = False,
	):
		"""Computes attention with the gfx950 kernels.  Same rules as the reference's
		GPU branch `_compute_triton` (:216-258): with Sq != Sk the mask is dropped,
		and a single query row is never causal."""
		if query.shape[1] != key.shape[1]:
			if query.shape[1] == 1:
				causal = False
			# (the 2-D validity mask of the reference; a 4-D boolean mask is turned into a bias by the operator and kept)
			if attention_mask is not None and len(attention_mask.shape) != 4:
				attention_mask = None

		if _is_jax_array(query):
			from ._jax_op import flash_attention as op  # XLA-FFI custom calls into the same C ABI

			if adjust_sharindgs:
				from ._jax_op import place_on_least_used_gpu

				query, key, value, bias, restore = place_on_least_used_gpu(query, key, value, bias)
		else:
			from ._hip_op import flash_attention as op  # torch tensors: ctypes into the C ABI

			restore = None

		attn = op(
			q=query,
			k=key,
			v=value,
			bias=bias,
			attention_mask=attention_mask,
			dropout_prob=dropout_prob,
			causal=causal,
			dropout_seed=dropout_seed,
			softmax_scale=self.config.softmax_scale,
		)
		if adjust_sharindgs and _is_jax_array(query) and restore is not None:
			attn = restore(attn)
		return attn

	def __repr__(self):
		return f"FlashAttention(platform={self.config.platform}, backend={self.config.backend})"

	__str__ = __repr__


def create_flash_attention(
	backend: tp.Optional[tp.Union[Backend, str]] = None,
	platform: tp.Optional[tp.Union[Platform, str]] = None,
	**kwargs,
) -> FlashAttention:
	"""Shorthand of the reference (:359-381): strings or enum members for backend and
	platform, remaining keywords go to `AttentionConfig`."""
	backend = Backend(backend) if isinstance(backend, str) else backend
	platform = Platform(platform) if isinstance(platform, str) else platform
	return FlashAttention(AttentionConfig(backend=backend, platform=platform, **kwargs))
