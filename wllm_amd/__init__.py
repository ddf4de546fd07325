"""A small, whole inference engine for one MI355X GPU.

Everything between a request's tokens and its next token: a typed
configuration and an architecture registry (`config`), weights by tensor name
(`weights`), layers assembled from parts (`parts`), a paged cache with
per-request block tables and state slots (`cache`), one step function over
mixed batches with a scheduler above it (`engine`), sampling (`sampling`), and
hand-written gfx950 kernels behind all of it (`csrc`, `kernels`).
"""

__version__ = "0.1.0"

from wllm_amd.config import register_architecture, resolve_architecture  # noqa: F401
from wllm_amd import architectures  # noqa: F401,E402  (registers the architectures)
