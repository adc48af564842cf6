from .step import CacheView, KVView, Span, StepContext, StepEntry, StepFunction

__all__ = ["CacheView", "KVView", "Span", "StepContext", "StepEntry", "StepFunction"]
