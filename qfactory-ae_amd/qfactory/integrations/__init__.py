"""Glue between the quantized linear and its callers' formats: the AutoGPTQ checkpoint tensors
(gptq_format) and the vLLM linear-method plugin (vllm_qfactory)."""
