"""Step function, scheduler, engine loop and command line."""
from .batch import BatchError, OutOfPages, StepBatch, build_step_batch
from .scheduler import Completion, Scheduler

__all__ = ["BatchError", "OutOfPages", "StepBatch", "build_step_batch", "Completion", "Scheduler", "LLMEngine",
           "ModelRunner", "Runtime", "resolve_kv_blocks"]


def __getattr__(name):
    # the engine and the runner need torch with a GPU; the scheduler and the batch do not
    if name in ("LLMEngine", "resolve_kv_blocks"):
        from . import engine
        return getattr(engine, name)
    if name == "ModelRunner":
        from .runner import ModelRunner
        return ModelRunner
    if name == "Runtime":
        from .runtime import Runtime
        return Runtime
    raise AttributeError(name)
