"""Architectures.  Every module of this package describes one and registers it when imported
(``registry.register_architecture``); ``discover()`` imports them all, so a new architecture is a new
file here (or, outside the package, any module that calls ``register_architecture`` before a model
is loaded, or an installed distribution with an entry point in the group
``flambeau_amd.architectures``)."""
import importlib
import pkgutil

from .decoder import DecoderModel, LayerSpec, ModelSpec, RunEntry

_discovered = False


def discover() -> None:
    global _discovered
    if _discovered:
        return
    _discovered = True
    for m in pkgutil.iter_modules(__path__):
        if m.name != "decoder":
            importlib.import_module(f"{__name__}.{m.name}")
    try:
        from importlib.metadata import entry_points
        eps = entry_points()
        group = eps.select(group="flambeau_amd.architectures") if hasattr(eps, "select") else eps.get("flambeau_amd.architectures", [])
        for ep in group:
            ep.load()
    except Exception:            # a broken third-party entry point must not break the built-in ones
        pass
