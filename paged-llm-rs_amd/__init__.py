"""A paged-KV inference engine for one GPU, native to the AMD MI355X (gfx950).

``config``    typed configurations and the architecture registry
``weights``   safetensors by tensor name, and the random-weights mode
``parts``     mixers, feed-forwards, norms, position encodings, blocks, the decoder
``cache``     pages, block tables, groups, state slots
``engine``    the step function, the scheduler, generation
``sampling``  greedy and temperature / top-k / top-p sampling
``csrc``      the HIP kernels and the native host runtime
"""

from .errors import (ConfigError, IoError, PagedLLMError, TensorError, UnsupportedError, WeightError)

__all__ = ["ConfigError", "IoError", "PagedLLMError", "TensorError", "UnsupportedError", "WeightError"]
__version__ = "0.1.0"
