"""atomserve_amd: a small, whole inference engine for one MI355X (gfx950).

From a model folder (config.json + safetensors) to generated tokens: typed
configuration and an architecture registry (`config`), weights by tensor name
(`weights`), layers assembled from parts (`parts`, `models`), a paged cache manager
(`cache`), one step function, a scheduler and the engine loop (`engine`), sampling
(`sampling`) and hand-written HIP kernels (`csrc`, loaded through `kernels`).
"""

__version__ = "0.1.0"
