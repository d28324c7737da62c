"""litellmengine_amd: a small, whole inference engine for one MI355X (gfx950).

From a model folder (config.json + safetensors) to generated tokens: typed
configuration and architecture registry (`config`), weights by name
(`weights`), model parts (`parts`) put together by an architecture (`models`),
a paged cache manager (`cache`), one step function with a scheduler above it
(`engine`), sampling (`sampling`), hand-written HIP kernels (`csrc`) and the
command-line entry points (`entrypoints`).
"""

__version__ = "0.1.0"
