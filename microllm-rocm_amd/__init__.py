"""A one-GPU inference engine for MI355X (gfx950), built around one step function.

Sub-packages, in the order a request passes them:
``config`` (typed configuration, architecture registry), ``weights`` (safetensors
by name, random weights), ``parts`` (norms, position encodings, mixers,
feed-forwards, blocks and the model they are put together into), ``cache``
(pages, block tables, state slots), ``engine`` (the step function, the scheduler,
generation and trace replay), ``sampling`` and ``ops`` (the bindings of the HIP
kernels under ``csrc``).
"""

__version__ = "0.1.0"
