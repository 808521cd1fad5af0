"""mini_infer_amd: a small, whole LLM inference engine for one AMD Instinct MI355X.

Model folder (config.json + safetensors) -> generated tokens on one GPU, on
hand-written HIP kernels (gfx950).  Entry points: `mini_infer_amd.LLM`,
`mini_infer_amd.engine.ModelRunner` + `ContinuousScheduler`, `python -m mini_infer_amd`.
"""

__version__ = "0.1.0"

# The names a user starts from, imported on first use (so that `import mini_infer_amd`
# alone stays light and the command line can parse its arguments before torch loads).
_LAZY = {
    "LLM": ("mini_infer_amd.engine.llm", "LLM"),
    "ModelRunner": ("mini_infer_amd.engine", "ModelRunner"),
    "ContinuousScheduler": ("mini_infer_amd.engine.scheduler", "ContinuousScheduler"),
    "Request": ("mini_infer_amd.engine.request", "Request"),
    "StepEntry": ("mini_infer_amd.engine", "StepEntry"),
    "SamplingParams": ("mini_infer_amd.sampling", "SamplingParams"),
    "ModelConfig": ("mini_infer_amd.config", "ModelConfig"),
    "EngineConfig": ("mini_infer_amd.config", "EngineConfig"),
}

__all__ = ["__version__", *_LAZY]


def __getattr__(name: str):
    try:
        module_name, attribute = _LAZY[name]
    except KeyError:
        raise AttributeError(f"module 'mini_infer_amd' has no attribute {name!r}") from None
    import importlib

    value = getattr(importlib.import_module(module_name), attribute)
    globals()[name] = value
    return value
