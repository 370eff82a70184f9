from .pinned import BatchUploader
from .profiler import OpProfiler, profiler, trace_enabled

__all__ = ["BatchUploader", "OpProfiler", "profiler", "trace_enabled"]
