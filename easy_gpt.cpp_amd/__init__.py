"""MI355X-native inference engine for the Qwen2 dense decoder.

From a model folder (config.json + model.safetensors) to next-token logits and
generated tokens on one GPU: typed configuration and architecture registry
(``config``), weights by tensor name (``weights``), layers assembled from parts
(``parts``, ``architectures``), a paged cache manager (``cache``), one step
function and a scheduler (``engine``), sampling (``sampling``) and hand-written
HIP kernels for gfx950 (``csrc``, bound in ``kernels``).
"""

__version__ = "0.1.0"
