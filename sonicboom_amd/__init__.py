"""sonicboom_amd: a small, whole inference library for one GPU (MI355X, gfx950).

Model folder (config.json + model.safetensors) in, generated tokens out:
typed configuration and architecture registry (``config``), weights by name
(``weights``), layers assembled from parts (``parts``), a paged KV cache with
per-sequence state (``cache``), one step function and a generation loop
(``engine``), sampling (``sampling``), hand-written HIP kernels (``csrc``,
``ops``).
"""
__version__ = "0.1.0"
