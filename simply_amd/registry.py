"""Name -> factory registries.

One `Registry` object per kind of thing that a configuration can name: whole
architectures, mixers, feed-forwards, norms, position encodings, block
arrangements, embeddings, heads and activations.  A registry is a plain dictionary with two rules taken from
simply/utils/registry.py:60-96: registering a name twice is an error, and asking
for an unknown name is an error that lists the known names.
"""
from __future__ import annotations

import importlib
import os
from typing import Any, Callable, Iterator

#: environment variable naming modules (comma-separated, importable) that register architectures and parts of
#: their own when they are imported: how a model that does not live in this package reaches the command line
#: and `bin/trace_run`
PLUGINS_ENV = "SIMPLY_AMD_PLUGINS"
_plugins_loaded = False


def load_plugins() -> None:
    """Imports the modules that $SIMPLY_AMD_PLUGINS names, once.  A registry does it by itself before it calls a
    name unknown."""
    global _plugins_loaded
    if _plugins_loaded:
        return
    _plugins_loaded = True
    for module in filter(None, (m.strip() for m in os.environ.get(PLUGINS_ENV, "").split(","))):
        try:
            importlib.import_module(module)
        except ImportError as exc:
            raise ImportError(f"${PLUGINS_ENV} names the module {module!r}, which cannot be imported: {exc}") from exc


class Registry:
    def __init__(self, kind: str):
        self.kind = kind
        self._entries: dict[str, Any] = {}

    def register(self, name: str, obj: Any = None, *, overwrite: bool = False):
        """`register(name, obj)` or, as a decorator, `@register(name)`."""

        def put(o):
            if name in self._entries and not overwrite:
                raise ValueError(f"duplicate {self.kind} name: {name!r}")
            self._entries[name] = o
            try:
                setattr(o, "__registered_name__", name)
            except (AttributeError, TypeError):
                pass
            return o

        return put if obj is None else put(obj)

    def unregister(self, name: str) -> None:
        self._entries.pop(name, None)

    def get(self, name: str) -> Any:
        if name not in self._entries:
            load_plugins()
        try:
            return self._entries[name]
        except KeyError:
            known = ", ".join(sorted(self._entries)) or "<none>"
            raise ValueError(f"unknown {self.kind} {name!r}; known: {known}") from None

    def build(self, name: str, *args, **kwargs) -> Any:
        """Calls the factory registered under `name` (get_instance in the reference)."""
        return self.get(name)(*args, **kwargs)

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def __iter__(self) -> Iterator[str]:
        return iter(sorted(self._entries))

    def keys(self):
        return sorted(self._entries)


#: architecture name (config.json "architectures"[0]) -> ArchitectureEntry
ARCHITECTURES = Registry("architecture")
#: part kinds, each name -> class with the interface given in simply_amd/parts/base.py
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("head")
#: activation name -> code of the gated product's epilogue (simply_amd/csrc/activations.h)
ACTIVATIONS = Registry("activation")
