from .runtime import Runtime, Workspace
from .step import Engine, LiveRequest, Span, StepContext, StepEntry, StepError

__all__ = ["Runtime", "Workspace", "Engine", "LiveRequest", "Span", "StepContext", "StepEntry", "StepError"]
