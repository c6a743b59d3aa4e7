"""An MI355X-native generation library for the Llama 2/3 dense decoder.

From a model folder (``config.json`` + safetensors) or seeded random weights to
generated tokens, through hand-written HIP kernels for gfx950:

    from gpt_fast_amd import Engine, generate
    engine = Engine.from_folder("path/to/model", dtype="bfloat16", max_tokens=8192)
    out = generate(engine, [[1, 2, 3], [4, 5]], max_new_tokens=16, temperature=0.0)
"""
from . import architectures as _architectures          # registers the known architectures
from .config.registry import (architecture, find_preset, known_architectures,
                              read_model_folder, register_architecture)
from .engine.batch import Entry
from .engine.step import Engine
from .parts.base import (register_block, register_feed_forward, register_mixer, register_norm,
                         register_position)
from .weights.random_init import write_random_model
from .engine.generate import GenerationResult, generate
from .engine.cli import main
from .sampling import SamplingParams
from . import config, weights, parts, cache, engine, sampling, ops


def _import_plugins():
    """Modules named in GPT_FAST_AMD_PLUGINS (comma-separated, importable names) are imported
    with the package, so that architectures and parts registered outside it are known to the
    command line and to the trace replay as well."""
    import importlib
    import os
    for name in filter(None, (n.strip() for n in os.environ.get("GPT_FAST_AMD_PLUGINS", "").split(","))):
        importlib.import_module(name)


_import_plugins()

