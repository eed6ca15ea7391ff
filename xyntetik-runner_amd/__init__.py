"""An inference engine for the Llama dense decoder on one AMD MI355X.

Everything between a request's tokens and its next token: typed configuration and an
architecture registry (``config``), safetensors weights and a random-weights mode
(``weights``), layers put together from parts (``parts``, ``architectures``), a paged
cache manager (``cache``), one step function with a scheduler above it (``engine``),
sampling (``sampling``), hand-written gfx950 kernels (``csrc``), a command line
(``cli``) and trace replay (``trace``).
"""
__version__ = "0.1.0"

from . import config, parts, architectures    # noqa: F401,E402  (fills the registries)
from .sampling import SamplingParams    # noqa: E402
from .llm import LLM    # noqa: E402

__all__ = ["LLM", "SamplingParams", "config", "parts", "architectures", "__version__"]
