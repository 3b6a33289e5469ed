"""Argument checks shared by the torch and the jax spelling of the operator.
Array-library neutral: only `.shape` and `.dtype` are looked at."""


def dtype_name(dt) -> str:
	"""'float16' / 'bfloat16' / ... for a torch, numpy or jax dtype."""
	return str(getattr(dt, "name", dt)).split(".")[-1]


def check_shapes(q, k, v, bias, attention_mask):
	"""Validation of `_fwd_attention_kernel_call` (_forward_triton.py:474-495) and
	`calc_bias_strides` (_utils.py:151-193), with the reference's messages."""
	batch, QSeq, nheads_q, head_dim = q.shape
	_, KSeq, nheads_kv, _ = k.shape
	expected_kv_shape = (batch, KSeq, nheads_kv, head_dim)
	if attention_mask is not None:
		assert bias is None, "Attention mask is not supported along with attention bias. Just use bias instead."
		assert QSeq == KSeq, "Attention mask is not supported with QSeq != KSeq"
	assert tuple(k.shape) == expected_kv_shape, (
		f"key shape is k.shape = {tuple(k.shape)} and we excepted it to be like expected_kv_shape = {expected_kv_shape}"
	)
	assert tuple(v.shape) == expected_kv_shape, (
		f"value shape is v.shape = {tuple(v.shape)} and we excepted it to be like expected_kv_shape = {expected_kv_shape}"
	)
	assert nheads_q % nheads_kv == 0, f"nheads_q = {nheads_q} is not divisible by nheads_kv ={nheads_kv}"
	assert dtype_name(q.dtype) == dtype_name(k.dtype) == dtype_name(v.dtype), "All tensors must have the same type"
	assert dtype_name(q.dtype) in ("float16", "bfloat16"), "Only support fp16 and bf16"
	if bias is not None:
		if bias.shape[2] != QSeq or bias.shape[3] != KSeq:
			raise ValueError(
				f"Bias tensor has incompatible sequence dimensions. "
				f"Expected shape [..., {QSeq}, {KSeq}], but got [..., {bias.shape[2]}, {bias.shape[3]}]. "
				f"Full bias shape: {tuple(bias.shape)}"
			)
		if bias.shape[0] not in (1, batch):
			raise ValueError(
				f"Batch dimension mismatch in bias tensor. "
				f"Expected either 1 (for broadcasting) or {batch} (batch size), "
				f"but got {bias.shape[0]}. Consider reshaping your bias tensor."
			)
		if bias.shape[1] not in (1, nheads_q) and not (bias.shape[1] == nheads_kv):
			raise ValueError(
				f"Head dimension mismatch in bias tensor. "
				f"Expected either 1 (for broadcasting) or {nheads_q} (number of heads), "
				f"but got {bias.shape[1]}. Check that your bias tensor matches the model configuration."
			)
