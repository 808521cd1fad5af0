from mini_infer_amd.engine.batch import StepEntry
from mini_infer_amd.engine.model_runner import ModelRunner

__all__ = ["ModelRunner", "StepEntry"]
