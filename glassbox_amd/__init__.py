"""glassbox_amd: a single-GPU inference engine for MI355X (gfx950).

    from glassbox_amd import Engine, generate, SamplerConfig
    engine = Engine("model_dir", dtype="bfloat16", max_tokens=8192)
    replies = generate(engine, [[1, 2, 3]], max_tokens=32, sampler=SamplerConfig(temperature=0.8, seed=1))
"""
__version__ = "0.1.0"

_LAZY = {
    "Engine": ".engine", "EngineError": ".engine", "Generator": ".engine", "generate": ".engine",
    "greedy": ".engine", "Scheduler": ".engine", "SchedulerConfig": ".engine",
    "SamplerConfig": ".sampling", "Sampler": ".sampling",
    "LlamaConfig": ".config", "config_from_dir": ".config", "register_architecture": ".config",
    "load_model": ".weights", "write_random_model": ".weights", "build_model": ".weights",
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        return getattr(importlib.import_module(_LAZY[name], __name__), name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
