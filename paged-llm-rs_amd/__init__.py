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



def __getattr__(name):
    # Engine and generate import torch and the native libraries; they load on first use.
    if name in ("Engine", "generate", "Replayer"):
        from . import engine
        return getattr(engine, name)
    if name in ("load_config", "register_architecture"):
        from . import config
        return getattr(config, name)
    if name == "write_random_model":
        from .weights import write_random_model
        return write_random_model
    raise AttributeError(name)


__all__ = ["Engine", "generate", "Replayer", "load_config", "register_architecture", "write_random_model",
           "ConfigError", "IoError", "PagedLLMError", "TensorError", "UnsupportedError", "WeightError"]
__version__ = "0.1.0"
