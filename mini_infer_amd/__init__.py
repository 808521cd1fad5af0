"""mini_infer_amd: a small, whole LLM inference engine for one AMD Instinct MI355X.

Model folder (config.json + safetensors) -> generated tokens on one GPU, on
hand-written HIP kernels.  See DESIGN.md at the repository root.
"""

__version__ = "0.1.0"
