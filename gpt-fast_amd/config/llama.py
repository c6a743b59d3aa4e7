"""Typed configuration of the Llama 2/3 dense decoder.

Field meanings are those of the reference's ``ModelArgs`` (model.py:21-42); the keys
are those of a checkpoint folder's ``config.json``.  No size lives in code: the named
presets below (the reference's ``transformer_configs``, model.py:60-82) are data that
produce the same ``config.json`` dictionaries a folder would hold.
"""
import json
import os
from dataclasses import dataclass
from typing import Optional, Tuple


def find_multiple(n: int, k: int) -> int:
    """Round ``n`` up to a multiple of ``k`` (reference model.py:16-19)."""
    return n if n % k == 0 else n + k - (n % k)


class ConfigError(ValueError):
    """A config.json that this library cannot run, with the reason."""


def _number(v):
    """An int stays an int (config.json round trip), anything else becomes a float."""
    return int(v) if isinstance(v, int) and not isinstance(v, bool) else float(v)


_ROPE_SCALING_KEYS = ("factor", "low_freq_factor", "high_freq_factor",
                      "original_max_position_embeddings")


@dataclass(frozen=True)
class LlamaConfig:
    hidden_size: int                      # dim            model.py:27
    num_hidden_layers: int                # n_layer        model.py:25
    num_attention_heads: int              # n_head         model.py:26
    num_key_value_heads: int              # n_local_heads  model.py:29,36-37
    head_dim: int                         # head_dim       model.py:30,42
    intermediate_size: int                # model.py:28,38-41
    vocab_size: int                       # model.py:24
    max_position_embeddings: int          # block_size     model.py:23
    rope_theta: float                     # rope_base      model.py:31
    rms_norm_eps: float                   # norm_eps       model.py:32
    rope_scaling: Optional[Tuple[Tuple[str, object], ...]] = None   # model.py:33
    tie_word_embeddings: bool = False
    bos_token_id: Optional[int] = None
    eos_token_id: Tuple[int, ...] = ()
    torch_dtype: str = "bfloat16"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, c: dict) -> "LlamaConfig":
        """Build from the keys of a ``config.json``.  Derivations follow the reference:
        kv heads default to the number of heads (model.py:36-37), the feed-forward width
        to ``find_multiple(int(2*4*dim/3), 256)`` (model.py:38-41), the head size to
        dim // heads (model.py:42) unless the file gives ``head_dim``."""
        def need(key):
            if key not in c or c[key] is None:
                raise ConfigError(f"config.json lacks '{key}'")
            return c[key]

        dim = int(need("hidden_size"))
        n_head = int(need("num_attention_heads"))
        n_kv = c.get("num_key_value_heads")
        n_kv = n_head if n_kv in (None, -1) else int(n_kv)
        inter = c.get("intermediate_size")
        inter = find_multiple(int(2 * (4 * dim) / 3), 256) if inter is None else int(inter)
        head_dim = c.get("head_dim")
        if head_dim is None:
            if dim % n_head:
                raise ConfigError(f"hidden_size {dim} is not a multiple of "
                                  f"num_attention_heads {n_head} and no head_dim is given")
            head_dim = dim // n_head
        head_dim = int(head_dim)

        for key in ("attention_bias", "mlp_bias"):
            if c.get(key):
                raise ConfigError(f"{key}=true: this decoder has no biases "
                                  f"(reference model.py:110,174-175,222-224)")
        act = c.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act='{act}': only 'silu' (reference model.py:227)")

        # newer folders keep the base and the scaling rule together under "rope_parameters"
        together = c.get("rope_parameters")
        if not isinstance(together, dict):
            together = {}
        theta = c.get("rope_theta", together.get("rope_theta", 10000.0))
        scaling = c.get("rope_scaling")
        if scaling is None and together:
            scaling = together
        if scaling is not None:
            kind = scaling.get("rope_type", scaling.get("type"))
            if kind in (None, "default"):
                scaling = None
            elif kind == "llama3":
                missing = [k for k in _ROPE_SCALING_KEYS if k not in scaling]
                if missing:
                    raise ConfigError(f"rope_scaling of type llama3 lacks {missing}")
                scaling = (("rope_type", "llama3"),) + tuple(
                    (k, _number(scaling[k])) for k in _ROPE_SCALING_KEYS)
            else:
                raise ConfigError(f"rope_scaling type '{kind}' is not supported "
                                  f"(known: llama3, default)")

        eos = c.get("eos_token_id")
        if eos is None:
            eos = ()
        elif isinstance(eos, int):
            eos = (eos,)
        else:
            eos = tuple(int(e) for e in eos)

        cfg = cls(
            hidden_size=dim, num_hidden_layers=int(need("num_hidden_layers")),
            num_attention_heads=n_head, num_key_value_heads=n_kv, head_dim=head_dim,
            intermediate_size=inter, vocab_size=int(need("vocab_size")),
            max_position_embeddings=int(c.get("max_position_embeddings", 2048)),
            rope_theta=float(theta),
            rms_norm_eps=float(c.get("rms_norm_eps", 1e-5)),
            rope_scaling=scaling,
            tie_word_embeddings=bool(c.get("tie_word_embeddings", False)),
            bos_token_id=c.get("bos_token_id"), eos_token_id=eos,
            torch_dtype=str(c.get("torch_dtype", c.get("dtype", "bfloat16"))),
        )
        cfg.validate()
        return cfg

    @classmethod
    def from_folder(cls, folder: str) -> "LlamaConfig":
        with open(os.path.join(folder, "config.json")) as f:
            return cls.from_dict(json.load(f))

    @classmethod
    def from_name(cls, name: str) -> "LlamaConfig":
        """A named preset; exact name first, then the longest preset name contained in
        ``name`` without regard to case (reference model.py:44-57)."""
        if name in PRESETS:
            return cls.from_dict(preset_dict(name))
        found = [p for p in PRESETS if p.lower() in str(name).lower()]
        if not found:
            raise ConfigError(f"no preset matches '{name}'; known: {sorted(PRESETS)}")
        found.sort(key=len, reverse=True)
        if len(found) > 1 and len(found[0]) == len(found[1]):
            raise ConfigError(f"'{name}' matches presets {found[0]} and {found[1]} equally")
        return cls.from_dict(preset_dict(found[0]))

    # ------------------------------------------------------------------ checking
    def validate(self) -> None:
        pos = ("hidden_size", "num_hidden_layers", "num_attention_heads",
               "num_key_value_heads", "head_dim", "intermediate_size", "vocab_size",
               "max_position_embeddings")
        for key in pos:
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads} (model.py:209-210)")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for rotary pairs")
        if not self.rms_norm_eps > 0:
            raise ConfigError("rms_norm_eps must be positive")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> dict:
        """The ``config.json`` dictionary of this configuration."""
        d = {
            "architectures": ["LlamaForCausalLM"], "model_type": "llama",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta, "rms_norm_eps": self.rms_norm_eps,
            "rope_scaling": None if self.rope_scaling is None else dict(self.rope_scaling),
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu", "attention_bias": False, "mlp_bias": False,
            "torch_dtype": self.torch_dtype,
        }
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id:
            d["eos_token_id"] = (self.eos_token_id[0] if len(self.eos_token_id) == 1
                                 else list(self.eos_token_id))
        return d


_LLAMA31_SCALING = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                    "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}

# Presets as data in the reference's own field names (model.py:60-82), plus the two tiny
# test shapes.  ``preset_dict`` turns one into config.json keys.
PRESETS = {
    "CodeLlama-7b-Python-hf": dict(block_size=16384, vocab_size=32000, n_layer=32, dim=4096,
                                   rope_base=1000000),
    "7B": dict(n_layer=32, n_head=32, dim=4096),
    "13B": dict(n_layer=40, n_head=40, dim=5120),
    "30B": dict(n_layer=60, n_head=52, dim=6656),
    "34B": dict(n_layer=48, n_head=64, dim=8192, vocab_size=32000, n_local_heads=8,
                intermediate_size=22016, rope_base=1000000),
    "70B": dict(n_layer=80, n_head=64, dim=8192, n_local_heads=8, intermediate_size=28672),
    "Mistral-7B": dict(n_layer=32, n_head=32, n_local_heads=8, dim=4096,
                       intermediate_size=14336, vocab_size=32000),
    "stories15M": dict(n_layer=6, n_head=6, dim=288),
    "stories110M": dict(n_layer=12, n_head=12, dim=768),
    "llama-3-8b": dict(block_size=8192, n_layer=32, n_head=32, n_local_heads=8, dim=4096,
                       intermediate_size=14336, vocab_size=128256, rope_base=500000),
    "llama-3-70b": dict(block_size=8192, n_layer=80, n_head=64, n_local_heads=8, dim=8192,
                        intermediate_size=28672, vocab_size=128256, rope_base=500000),
    "llama-3.1-8b": dict(block_size=131072, n_layer=32, n_head=32, n_local_heads=8, dim=4096,
                         intermediate_size=14336, vocab_size=128256, rope_base=500000,
                         rope_scaling=_LLAMA31_SCALING),
    "llama-3.1-70b": dict(block_size=131072, n_layer=80, n_head=64, n_local_heads=8,
                          dim=8192, intermediate_size=28672, vocab_size=128256,
                          rope_base=500000, rope_scaling=_LLAMA31_SCALING),
    "llama-3.1-405b": dict(block_size=131072, n_layer=126, n_head=128, n_local_heads=8,
                           dim=16384, intermediate_size=53248, vocab_size=128256,
                           rope_base=500000, rope_scaling=_LLAMA31_SCALING),
    "tiny-llama-a": dict(block_size=64, n_layer=2, n_head=4, n_local_heads=4, dim=64,
                         intermediate_size=176, vocab_size=256, rope_base=10000,
                         norm_eps=1e-5),
    "tiny-llama-b": dict(block_size=128, n_layer=3, n_head=6, n_local_heads=2, dim=192,
                         intermediate_size=512, vocab_size=384, rope_base=500000,
                         norm_eps=1e-6,
                         rope_scaling={"rope_type": "llama3", "factor": 8.0,
                                       "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                       "original_max_position_embeddings": 32}),
}

# Defaults of the reference's ModelArgs (model.py:23-33) for fields a preset leaves out.
_MODELARGS_DEFAULTS = dict(block_size=2048, vocab_size=32000, n_layer=32, n_head=32, dim=4096,
                           intermediate_size=None, n_local_heads=-1, rope_base=10000,
                           norm_eps=1e-5, rope_scaling=None)


def preset_dict(name: str) -> dict:
    """The ``config.json`` dictionary of a preset."""
    a = dict(_MODELARGS_DEFAULTS)
    a.update(PRESETS[name])
    return {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": a["dim"], "num_hidden_layers": a["n_layer"],
        "num_attention_heads": a["n_head"], "num_key_value_heads": a["n_local_heads"],
        "intermediate_size": a["intermediate_size"], "vocab_size": a["vocab_size"],
        "max_position_embeddings": a["block_size"], "rope_theta": float(a["rope_base"]),
        "rms_norm_eps": a["norm_eps"], "rope_scaling": a["rope_scaling"],
    }
