"""One registry from an architecture's name to how its model is made.

The key is ``architectures[0]`` of config.json (or its ``architecture``), with ``model_type`` as a second chance
(the reference keys on ``model_type`` alone: kvcore/model/model_loader/
default_loader.py:32-36,64-70).  An entry holds a parser from the raw config mapping to
a typed configuration and a function from that configuration to a ``ModelSpec``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping

from kvcore_amd.models.spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[[Mapping[str, Any]], Any]
    build_spec: Callable[[Any], ModelSpec]
    # fills in what config.json leaves to the checkpoint's tensor shapes: (config mapping, a
    # function from tensor name to shape or None) -> config mapping; None: nothing to fill in
    complete_config: Callable[[Mapping[str, Any], Callable[[str], Any]], Mapping[str, Any]] | None = None


MODEL_REGISTRY: dict[str, Architecture] = {}


def register_architecture(name: str, parse_config: Callable[[Mapping[str, Any]], Any],
                          build_spec: Callable[[Any], ModelSpec], *, aliases: tuple[str, ...] = (),
                          replace: bool = False, complete_config=None) -> None:
    arch = Architecture(name, parse_config, build_spec, complete_config)
    for key in (name, *aliases):
        if key in MODEL_REGISTRY and not replace:
            raise ValueError(f"architecture {key!r} is already registered")
        MODEL_REGISTRY[key] = arch


def unregister_architecture(name: str) -> None:
    MODEL_REGISTRY.pop(name, None)


def resolve_architecture(config: Mapping[str, Any]) -> Architecture:
    names = list(config.get("architectures") or [])
    if config.get("architecture"):  # some configurations name one architecture, in the singular
        names.append(config["architecture"])
    if config.get("model_type"):
        names.append(config["model_type"])
    for name in names:
        if name in MODEL_REGISTRY:
            return MODEL_REGISTRY[name]
    raise ValueError(
        f"Unsupported architecture {names or None!r}. Supported: {sorted(MODEL_REGISTRY)}"
    )


def _register_builtin() -> None:
    from kvcore_amd.config.model_config import LlamaConfig
    from kvcore_amd.models.llama import llama_spec

    register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, llama_spec, aliases=("llama",))

    from kvcore_amd.config.dirulorn_config import DirulornConfig
    from kvcore_amd.models.dirulorn import dirulorn_spec

    register_architecture("Dirulorn", DirulornConfig.from_dict, dirulorn_spec)

    from kvcore_amd.config.vovalix_config import VovalixConfig, complete_from_tensor_shapes
    from kvcore_amd.models.vovalix import vovalix_spec

    register_architecture("Vovalix", VovalixConfig.from_dict, vovalix_spec,
                          complete_config=complete_from_tensor_shapes)

    from kvcore_amd.config.tazunex_config import TazunexConfig
    from kvcore_amd.models.tazunex import tazunex_spec

    register_architecture("Tazunex", TazunexConfig.from_dict, tazunex_spec)

    from kvcore_amd.config.darovik_config import DarovikConfig
    from kvcore_amd.models.darovik import darovik_spec

    register_architecture("Darovik", DarovikConfig.from_dict, darovik_spec)


_register_builtin()
