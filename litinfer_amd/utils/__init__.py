from .profiler import OpProfiler, profiler, trace_enabled

__all__ = ["OpProfiler", "profiler", "trace_enabled"]
