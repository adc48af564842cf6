from .step import KVView, Span, StepContext, StepEntry, StepFunction

__all__ = ["KVView", "Span", "StepContext", "StepEntry", "StepFunction"]
