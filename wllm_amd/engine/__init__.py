from wllm_amd.engine.batch import PageView, StepContext, StepEntry, Workspace
from wllm_amd.engine.runner import ModelRunner, StepError

__all__ = ["PageView", "StepContext", "StepEntry", "Workspace", "ModelRunner", "StepError"]
