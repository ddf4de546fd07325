from wllm_amd.parts import attention, blocks, feed_forward, norms, positions  # noqa: F401  (register the kinds)
from wllm_amd.parts.model import (CausalLM, build_model, load_model, resolve_dtype, write_random_model_folder,
                                   write_random_model_from_config_json)
from wllm_amd.parts.registry import (
    build_block, build_feed_forward, build_mixer, build_norm, build_position,
    register_block, register_feed_forward, register_mixer, register_norm, register_position,
)

__all__ = [
    "CausalLM", "build_model", "load_model", "resolve_dtype", "write_random_model_folder",
    "write_random_model_from_config_json",
    "build_block", "build_feed_forward", "build_mixer", "build_norm", "build_position",
    "register_block", "register_feed_forward", "register_mixer", "register_norm", "register_position",
]
