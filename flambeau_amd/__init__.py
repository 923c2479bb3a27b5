"""flambeau_amd: a small, whole inference engine for one MI355X.

    from flambeau_amd import generate
    out = generate("path/to/model", [[1, 5, 9]], max_new_tokens=16)

The model class is chosen by the folder's config.json.  Everything on the device runs in
hand-written HIP kernels for gfx950, compiled at first use; there is no CPU path.
"""
__version__ = "0.1.0"

_LAZY = {
    "generate": "engine", "LLMEngine": "engine", "EngineOptions": "engine", "ModelRunner": "engine",
    "StepEntry": "engine", "load_model": "engine", "random_model": "engine",
    "SamplingParams": "sampling",
    "write_random_model": "weights",
    "register_architecture": "registry", "find_architecture": "registry", "known_architectures": "registry",
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        return getattr(importlib.import_module(f"{__name__}.{_LAZY[name]}"), name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
