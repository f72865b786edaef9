"""A Qwen3 dense inference engine for MI355X: configuration, weights, parts, paged cache,
one step function, scheduler, sampling, on hand-written gfx950 kernels.

Importing the package touches neither the GPU nor the kernel library; the first kernel call
loads (and, if need be, builds) the library.
"""
__version__ = "0.1.0"

_LAZY = {
    "Runtime": "api", "generate": "api", "sampling_params": "api",
    "SamplingParams": "sampling.sampler",
    "Engine": "engine.engine", "StepEntry": "engine.engine",
    "Scheduler": "engine.scheduler", "SchedulerPolicy": "engine.scheduler",
    "load_model": "runtime", "random_model": "runtime",
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        return getattr(importlib.import_module(f"{__name__}.{_LAZY[name]}"), name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
