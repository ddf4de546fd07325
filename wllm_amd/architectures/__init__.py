"""Architectures: each module turns its typed configuration into a ModelPlan
and registers itself under the names config.json may carry."""
from wllm_amd.architectures import gemma  # noqa: F401  (registers GemmaForCausalLM)
from wllm_amd.architectures.gemma_config import GemmaConfig  # noqa: F401
