"""denno-beta_amd: a small, whole inference engine for one GPU (AMD MI355X, gfx950).

Everything between a request's tokens and its next token: typed configuration and a
registry of architectures (`config`), weights from safetensors (`weights`), layers put
together from parts (`parts`, `models`), a paged cache (`cache`), one step function with a
scheduler above it (`engine`), sampling (`sampling`), and hand-written HIP kernels
(`kernels`, sources under `csrc/`).
"""
__version__ = "0.1.0"
