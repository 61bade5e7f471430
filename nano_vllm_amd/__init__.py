"""A small inference engine for one MI355X (gfx950): Qwen3 dense, from a model folder to
generated tokens, on hand-written HIP kernels."""
__version__ = "0.1.0"

from .sampling.params import SamplingParams   # noqa: E402
from .llm import LLM                           # noqa: E402

__all__ = ["LLM", "SamplingParams", "__version__"]
