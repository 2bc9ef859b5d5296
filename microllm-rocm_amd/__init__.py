"""A one-GPU inference engine for MI355X (gfx950), built around one step function.

Sub-packages, in the order a request passes them:
``config`` (typed configuration, architecture registry), ``weights`` (safetensors
by name, random weights), ``parts`` (norms, position encodings, mixers,
feed-forwards, blocks and the model they are put together into), ``cache``
(pages, block tables, state slots), ``engine`` (the step function, the scheduler,
generation and trace replay), ``sampling`` and ``ops`` (the bindings of the HIP
kernels under ``csrc``).

    engine = Engine.from_folder("model_dir", dtype="bfloat16", max_tokens=8192)
    tokens = generate(engine, [[1, 2, 3]], GenerationConfig(max_new_tokens=16, temperature=0.0))
"""

__version__ = "0.1.0"

from .config import ConfigError, Qwen2Config, load_config, register_architecture  # noqa: E402
from .engine import (Engine, GenerationConfig, Scheduler, StepEntry, generate,  # noqa: E402
                     generate_serial)
from .sampling import SamplingParams  # noqa: E402
from .weights import WeightsError, write_model_folder  # noqa: E402

__all__ = ["ConfigError", "Qwen2Config", "load_config", "register_architecture", "Engine", "GenerationConfig",
           "Scheduler", "StepEntry", "generate", "generate_serial", "SamplingParams", "WeightsError",
           "write_model_folder"]
