"""Host-side mirror of the reference facade (flash_attention.py:74-212, 359-381):
enums, defaults, validation and error messages.  No GPU."""

import pytest
import torch

import jax_flash_attn2 as fa
from jax_flash_attn2 import _hip_op
from jax_flash_attn2.flash_attention import AttentionConfig, Backend, FlashAttention, Platform, create_flash_attention


def test_enums_and_defaults():
	assert [b.value for b in Backend] == ["gpu", "tpu", "cpu"]
	assert [p.value for p in Platform] == ["triton", "pallas", "jax", "hip"]
	c = AttentionConfig(backend=Backend.GPU)
	assert (c.blocksize_q, c.blocksize_k, c.softmax_scale, c.platform) == (128, 128, None, Platform.HIP)
	assert AttentionConfig(backend=Backend.CPU).platform == Platform.JAX
	assert AttentionConfig(backend=Backend.TPU).platform == Platform.PALLAS
	assert set(fa.__all__) >= {"AttentionConfig", "Backend", "Platform", "FlashAttention", "create_flash_attention"}


@pytest.mark.parametrize(
	"backend,platform,ok",
	[("gpu", "hip", True), ("gpu", "triton", True), ("gpu", "pallas", True), ("gpu", "jax", True), ("cpu", "jax", True),
	 ("tpu", "jax", True), ("tpu", "pallas", True), ("cpu", "triton", False), ("cpu", "hip", False), ("tpu", "hip", False),
	 ("cpu", "pallas", False)],
)
def test_backend_platform_pairs(backend, platform, ok):
	if ok:
		a = create_flash_attention(backend, platform, softmax_scale=0.5)
		assert a.config.softmax_scale == 0.5
		assert "FlashAttention(platform=" in repr(a)
	else:
		with pytest.raises(ValueError, match="Invalid backend-platform combination"):
			create_flash_attention(backend, platform)
	with pytest.raises(ValueError):
		create_flash_attention("gpu", "cuda")


def test_head_divisibility_and_bias_heads():
	a = create_flash_attention("gpu", "hip")
	q = torch.zeros(1, 8, 6, 64, dtype=torch.bfloat16)
	k = torch.zeros(1, 8, 4, 64, dtype=torch.bfloat16)
	with pytest.raises(ValueError, match=r"Query heads \(6\) must be divisible by key/value heads \(4\)"):
		a(q, k, k)
	k2 = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16)
	with pytest.raises(ValueError, match="Incompatible bias shape. Got 3 heads, expected 6, 2, or 1"):
		a(q, k2, k2, bias=torch.zeros(1, 3, 8, 8))
	for h in (1, 2, 6):
		assert a._handle_bias(torch.zeros(1, h, 8, 8), 6, 2).shape[1] == h
	assert a._handle_bias(None, 6, 2) is None
	kk, vv = FlashAttention.repeat_kv_heads(torch.arange(4.0).reshape(1, 1, 2, 2), torch.zeros(1, 1, 2, 2), 3)
	assert kk.shape == (1, 1, 6, 2) and torch.equal(kk[0, 0, :, 0], torch.tensor([0.0, 0, 0, 2, 2, 2]))


def test_operator_shape_checks():
	q = torch.zeros(2, 16, 4, 64, dtype=torch.bfloat16)
	k = torch.zeros(2, 16, 2, 64, dtype=torch.bfloat16)
	with pytest.raises(AssertionError, match="Only support fp16 and bf16"):
		_hip_op.check_shapes(q.float(), k.float(), k.float(), None, None)
	with pytest.raises(AssertionError, match="All tensors must have the same type"):
		_hip_op.check_shapes(q, k.half(), k, None, None)
	with pytest.raises(AssertionError, match="value shape is"):
		_hip_op.check_shapes(q, k, k[:, :8], None, None)
	with pytest.raises(AssertionError, match="Attention mask is not supported along with attention bias"):
		_hip_op.check_shapes(q, k, k, torch.zeros(2, 1, 16, 16), torch.ones(2, 16))
	with pytest.raises(AssertionError, match="QSeq != KSeq"):
		_hip_op.check_shapes(q[:, :8], k, k, None, torch.ones(2, 16))
	with pytest.raises(ValueError, match="incompatible sequence dimensions"):
		_hip_op.check_shapes(q, k, k, torch.zeros(2, 1, 16, 15), None)
	with pytest.raises(ValueError, match="Batch dimension mismatch"):
		_hip_op.check_shapes(q, k, k, torch.zeros(3, 1, 16, 16), None)
	with pytest.raises(ValueError, match="Head dimension mismatch"):
		_hip_op.check_shapes(q, k, k, torch.zeros(2, 3, 16, 16), None)
	_hip_op.check_shapes(q, k, k, torch.zeros(1, 4, 16, 16), None)


def test_unbuilt_platforms_say_so():
	q = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16)
	with pytest.raises(NotImplementedError):
		create_flash_attention("cpu", "jax")(q, q, q)
	with pytest.raises(NotImplementedError):
		create_flash_attention("tpu", "pallas")(q, q, q)


def test_package_exports_the_names_of_the_reference():
	"""jax_flash_attn2/__init__.py:23-35 of the reference: every public name exists here; the two pure-XLA
	implementations are names that say they are not part of this package."""
	import jax_flash_attn2 as pkg

	for name in ("AttentionConfig", "Backend", "FlashAttention", "Platform", "create_flash_attention",
	             "triton_flash_attention", "jax_flash_attention", "basic_attention_refrence"):
		assert hasattr(pkg, name) and name in pkg.__all__, name
	assert pkg.triton_flash_attention is pkg.hip_flash_attention
	for fn in (pkg.jax_flash_attention, pkg.basic_attention_refrence):
		with pytest.raises(NotImplementedError, match="HIP"):
			fn(None, None, None)


def test_kernel_head_dim_padding_rule():
	torch = pytest.importorskip("torch")
	from jax_flash_attn2 import _hip_op

	assert [_hip_op._kernel_head_dim(d) for d in (16, 64, 65, 128, 129, 256)] == [64, 64, 128, 128, 256, 256]
	with pytest.raises(ValueError):
		_hip_op._kernel_head_dim(257)
	x = torch.ones(1, 2, 3, 80)
	y = _hip_op._pad_d(x, 128)
	assert y.shape == (1, 2, 3, 128) and float(y[..., 80:].abs().sum()) == 0.0 and _hip_op._pad_d(y, 128) is y
