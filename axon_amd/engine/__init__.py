from .runtime import Runtime, Workspace
from .step import Engine, LiveRequest, PendingPicks, Span, StepContext, StepEntry, StepError

__all__ = ["Runtime", "Workspace", "Engine", "LiveRequest", "PendingPicks", "Span", "StepContext", "StepEntry", "StepError"]
