"""The step function, the scheduler above it, request tasks and trace replay."""
from .context import LayerCacheView, StepContext, Workspace
from .engine import Engine, StepEntry

__all__ = ["Engine", "StepEntry", "LayerCacheView", "StepContext", "Workspace"]
