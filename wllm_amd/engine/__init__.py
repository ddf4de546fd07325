from wllm_amd.engine.batch import PageView, StepContext, StepEntry, Workspace
from wllm_amd.engine.llm import LLM, RequestOutput
from wllm_amd.engine.request import Request, RequestStatus
from wllm_amd.engine.runner import ModelRunner, StepError
from wllm_amd.engine.scheduler import RequestRefused, Scheduler

__all__ = ["PageView", "StepContext", "StepEntry", "Workspace", "LLM", "RequestOutput", "Request",
           "RequestStatus", "ModelRunner", "StepError", "RequestRefused", "Scheduler"]
