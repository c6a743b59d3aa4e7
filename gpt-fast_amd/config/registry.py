"""The one registry from an architecture's name to its model.

An :class:`Architecture` bundles what is particular to one model family: how its
``config.json`` is read into a typed configuration, how that configuration becomes a
:class:`~.spec.ModelPlan`, and how the tensors of its checkpoint files map to the
plan's parameters.  Everything else in the library is shared.

The reference picks its one model class by the checkpoint folder's name
(generate.py:222, model.py:44-57, 148-150); here ``config.json`` names it through
``architectures[0]`` or ``model_type``.
"""
import json
import os
from dataclasses import dataclass
from typing import Callable, Dict, Tuple


class UnknownArchitecture(KeyError):
    pass


@dataclass(frozen=True)
class Architecture:
    names: Tuple[str, ...]                      # e.g. ("LlamaForCausalLM", "llama")
    read_config: Callable[[dict], object]       # config.json dict -> typed configuration
    plan: Callable[[object], object]            # typed configuration -> ModelPlan
    bindings: Callable[[object], list]          # typed configuration -> [weights.Binding]
    config_dict: Callable[[object], dict]       # typed configuration -> config.json dict
    presets: Callable[[str], object] = None     # preset name -> typed configuration
    # typed configuration -> further CheckpointLayouts under which the same parameters may
    # be stored (other tensor names); the loader takes the one that fits the files' names
    other_layouts: Callable[[object], tuple] = None
    # typed configuration -> every size and constant under a short name, flat (numbers and
    # strings only), for reports and benchmark records
    describe: Callable[[object], dict] = None
    # the config.json key that holds the number of layers (a benchmark may run fewer)
    layer_count_key: str = "num_hidden_layers"

    def layouts(self, config) -> tuple:
        """Every layout a checkpoint of ``config`` may have; the first is the one that
        random weights are written in."""
        more = tuple(self.other_layouts(config)) if self.other_layouts is not None else ()
        return (self.bindings(config),) + more


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> Architecture:
    for name in arch.names:
        _ARCHITECTURES[name] = arch
    return arch


def known_architectures():
    return sorted(_ARCHITECTURES)


def architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise UnknownArchitecture(
            f"unknown architecture '{name}'; known: {known_architectures()}") from None


def find_preset(name: str, architecture_name: str = None):
    """(architecture, typed configuration) of a named preset.  With ``architecture_name``
    that architecture's presets are asked; else every registered architecture's, and the
    name must be known to exactly one of them."""
    if architecture_name is not None:
        arch = architecture(architecture_name)
        if arch.presets is None:
            raise UnknownArchitecture(f"architecture '{architecture_name}' has no presets")
        return arch, arch.presets(name)
    found, errors = [], []
    for arch in {id(a): a for a in _ARCHITECTURES.values()}.values():
        if arch.presets is None:
            continue
        try:
            found.append((arch, arch.presets(name)))
        except (KeyError, ValueError) as e:
            errors.append(str(e))
    if not found:
        raise UnknownArchitecture(f"no architecture has a preset '{name}': " + "; ".join(errors))
    if len(found) > 1:
        raise UnknownArchitecture(
            f"preset '{name}' is known to several architectures "
            f"({', '.join(a.names[0] for a, _ in found)}); name one")
    return found[0]


def architecture_of(config_json: dict) -> Architecture:
    """The architecture that a ``config.json`` dictionary names."""
    names = list(config_json.get("architectures") or [])
    if config_json.get("model_type"):
        names.append(config_json["model_type"])
    if not names:
        raise UnknownArchitecture(
            "config.json has neither 'architectures' nor 'model_type'; "
            f"known: {known_architectures()}")
    for name in names:
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
    raise UnknownArchitecture(
        f"unknown architecture {names}; known: {known_architectures()}")


def read_model_folder(folder: str):
    """(architecture, typed configuration) of a model folder."""
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{path}: a model folder needs a config.json")
    with open(path) as f:
        raw = json.load(f)
    arch = architecture_of(raw)
    return arch, arch.read_config(raw)
