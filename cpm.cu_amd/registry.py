"""One registry from an architecture's name (config.json ``architectures[0]``) to its model.

An architecture brings: its typed configuration class, a function that builds the
model (parts and schedule) from a configuration, the options that function
understands, and the checkpoint's peculiarities (fused tensors to split, tensors
to ignore, options that the checkpoint decides).  The reference chooses the model
class from the same config key (cpmcu/common/utils.py:33-64).  Nothing outside
an architecture's own file names its options or its configuration's fields.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Iterable, List, Mapping, Optional, Sequence


@dataclass(frozen=True)
class Flag:
    """A front-end flag that an architecture declares: ``name`` is the keyword of ``LLM(...)`` and, with dashes
    or underscores, the command-line option; ``kind`` is int, float, str or bool (a boolean takes true/false
    values on the command line)."""
    name: str
    kind: type = int
    help: str = ""
    group: str = "Model Configuration"


@dataclass
class Architecture:
    name: str
    config_class: type
    build: Callable                                  # (config, **options) -> model
    options: Dict[str, Any] = field(default_factory=dict)   # the options ``build`` understands, with their defaults
    split_fused: Optional[Callable] = None           # (config, name, tensor) -> [(name, tensor)] or None
    ignore_tensor: Optional[Callable] = None         # (config, name) -> bool
    # (config, names of the checkpoint's tensors) -> options that the checkpoint decides (e.g. tied embeddings
    # when the head's tensor is absent); explicit options win over them
    checkpoint_options: Optional[Callable] = None
    # (config, flags) -> (config, options): the front end's flags (the reference's command-line and ``LLM``
    # argument names) as this architecture understands them; flags it does not know must be refused
    apply_flags: Optional[Callable] = None
    # the flags ``apply_flags`` knows, as the front ends should offer them (command-line options, keywords of
    # ``LLM``); and the command line's --model-type names with the flags each one sets
    flags: Sequence[Flag] = ()
    model_types: Mapping[str, Mapping[str, Any]] = field(default_factory=dict)

    def build_model(self, config, options: Optional[Mapping[str, Any]] = None,
                    checkpoint_names: Optional[Iterable[str]] = None):
        """The model for ``config``: defaults, then what the checkpoint decides, then the given options."""
        opts = dict(self.options)
        if checkpoint_names is not None and self.checkpoint_options is not None:
            opts.update(self.checkpoint_options(config, set(checkpoint_names)))
        for k, v in (options or {}).items():
            if k not in self.options:
                raise ValueError(f"architecture '{self.name}' has no option '{k}' (it has: {sorted(self.options) or 'none'})")
            opts[k] = v
        return self.build(config, **opts)

    def with_flags(self, config, flags: Optional[Mapping[str, Any]]):
        """(config, options) after the front end's flags; flags that are None or absent change nothing."""
        given = {k: v for k, v in (flags or {}).items() if v is not None}
        if self.apply_flags is None:
            switched_on = sorted(k for k, v in given.items() if v is not False)
            if switched_on:
                raise ValueError(f"architecture '{self.name}' takes no flags, got {switched_on}")
            return config, {}
        return self.apply_flags(config, given) if given else (config, {})


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, replace: bool = False):
    if arch.name in _ARCHITECTURES and not replace and _ARCHITECTURES[arch.name] is not arch:
        raise ValueError(f"architecture '{arch.name}' is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def unregister_architecture(name: str):
    _ARCHITECTURES.pop(name, None)


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise KeyError(f"unknown architecture '{name}' (registered: {sorted(_ARCHITECTURES)})") from None


def architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


def declared_flags() -> List[Flag]:
    """Every flag that a registered architecture declares, once by name (the first declaration's help stands)."""
    seen: Dict[str, Flag] = {}
    for name in sorted(_ARCHITECTURES):
        for f in _ARCHITECTURES[name].flags:
            if f.name in seen and seen[f.name].kind is not f.kind:
                raise ValueError(f"flag '{f.name}' is declared as {seen[f.name].kind.__name__} and as {f.kind.__name__}")
            seen.setdefault(f.name, f)
    return list(seen.values())


def declared_model_types() -> List[str]:
    return sorted({t for a in _ARCHITECTURES.values() for t in a.model_types})
