from .context import StepContext
from .engine import Engine, parse_dtype
from .layout import StepEntry, StepLayout, build_step_layout

__all__ = ["Engine", "StepContext", "StepEntry", "StepLayout", "build_step_layout", "parse_dtype"]
