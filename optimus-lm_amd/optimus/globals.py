profiler = None
