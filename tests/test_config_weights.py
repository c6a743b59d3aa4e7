"""Configuration, registry, safetensors reading, weight errors and the random-weights
mode.  No GPU."""
import json
import os

import pytest
import torch

import plain_llama as plain
import util

import gpt_fast_amd as gfa
from gpt_fast_amd.config.llama import ConfigError, LlamaConfig, preset_dict
from gpt_fast_amd.config.registry import UnknownArchitecture, architecture_of
from gpt_fast_amd.weights.bindings import WeightsError, load_parameters
from gpt_fast_amd.weights.safetensors_io import SafetensorsFile, write_safetensors


def test_config_from_keys_and_derivations():
    c = LlamaConfig.from_dict(util.TINY_B)
    assert (c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (192, 6, 2, 32)
    assert c.intermediate_size == 512 and c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0
    assert dict(c.rope_scaling)["original_max_position_embeddings"] == 32
    # derived values of the reference (model.py:36-42)
    d = LlamaConfig.from_dict(dict(hidden_size=4096, num_attention_heads=32,
                                   num_hidden_layers=2, vocab_size=100))
    assert d.num_key_value_heads == 32 and d.head_dim == 128 and d.intermediate_size == 11008
    # a given intermediate_size and head_dim are honoured
    assert LlamaConfig.from_dict(util.TINY_A).intermediate_size == 176
    assert LlamaConfig.from_dict(util.TINY_C).head_dim == 48
    # round trip through config.json keys
    assert LlamaConfig.from_dict(c.to_dict()) == c
    # the base and the scaling rule kept together under one key read the same
    moved = {k: v for k, v in util.TINY_B.items() if k not in ("rope_theta", "rope_scaling")}
    moved["rope_parameters"] = dict(util.TINY_B["rope_scaling"], rope_theta=util.TINY_B["rope_theta"])
    assert LlamaConfig.from_dict(moved) == c
    plain_rope = {k: v for k, v in util.TINY_A.items() if k not in ("rope_theta", "rope_scaling")}
    plain_rope["rope_parameters"] = {"rope_type": "default", "rope_theta": 12345.0}
    e = LlamaConfig.from_dict(plain_rope)
    assert e.rope_theta == 12345.0 and e.rope_scaling is None


def test_presets_match_reference_registry():          # model.py:44-82
    c = LlamaConfig.from_name("llama-3.1-8b")
    assert (c.num_hidden_layers, c.hidden_size, c.intermediate_size, c.vocab_size) == (32, 4096, 14336, 128256)
    assert dict(c.rope_scaling)["factor"] == 8.0 and c.max_position_embeddings == 131072
    # fuzzy match: longest preset name contained in the given name wins
    assert LlamaConfig.from_name("Meta-Llama-3.1-70B-Instruct").num_hidden_layers == 80
    assert LlamaConfig.from_name("Mistral-7B-v0.1").num_key_value_heads == 8
    assert LlamaConfig.from_name("llama-2-7b-chat-hf").intermediate_size == 11008
    with pytest.raises(ConfigError):
        LlamaConfig.from_name("nothing-like-it")


@pytest.mark.parametrize("patch,word", [
    ({"attention_bias": True}, "attention_bias"), ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"), ({"rope_scaling": {"rope_type": "yarn"}}, "yarn"),
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "even"),
    ({"hidden_size": None}, "hidden_size"),
])
def test_config_refusals(patch, word):
    raw = dict(util.TINY_A)
    raw.update(patch)
    with pytest.raises(ConfigError, match=word):
        LlamaConfig.from_dict(raw)


def test_registry_names_the_model():
    assert architecture_of({"architectures": ["LlamaForCausalLM"]}) is gfa.architecture("llama")
    assert architecture_of({"model_type": "llama"}) is gfa.architecture("LlamaForCausalLM")
    with pytest.raises(UnknownArchitecture, match="LlamaForCausalLM"):
        architecture_of({"architectures": ["SomethingElse"]})
    with pytest.raises(UnknownArchitecture):
        architecture_of({})


def test_plan_is_data():
    arch = gfa.architecture("llama")
    plan = arch.plan(LlamaConfig.from_dict(util.TINY_B))
    assert len(plan.layers) == 3 and [r.layer for r in plan.order] == [0, 1, 2]
    m = plan.layers[1].mixer
    assert (m.n_heads, m.n_kv_heads, m.head_dim, m.position.base) == (6, 2, 32, 500000.0)
    assert plan.layers[0].mixer_norm.eps == 1e-6 and plan.layers[2].feed_forward.hidden == 512


def test_safetensors_round_trip(tmp_path):
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16),
         "c": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, t)
    f = SafetensorsFile(path)
    assert f.entries["b"] == ("BF16", (7,))
    for k, v in t.items():
        assert torch.equal(f.tensor(k), v)
    # the plain reader and the safetensors package read the same file
    mine = plain.read_safetensors(path)
    assert torch.equal(mine["a"], t["a"]) and torch.equal(mine["b"], t["b"].float())
    from safetensors.torch import load_file
    theirs = load_file(path)
    assert all(torch.equal(theirs[k], v) for k, v in t.items())


def _folder(tmp_path, name="A", dtype="float32"):
    return util.make_folder(tmp_path, name, seed=1, dtype=dtype)


def test_loader_fuses_and_permutes_like_the_converter(tmp_path):
    folder = _folder(tmp_path, "B")
    arch, cfg = gfa.read_model_folder(folder)
    params = load_parameters(folder, arch.bindings(cfg), "float32", None)
    pcfg, w = plain.load_folder(folder)
    assert torch.equal(params["layers.1.attention.wqkv"], w["layers.1.attention.wqkv.weight"])
    assert torch.equal(params["layers.2.feed_forward.w13"][:512], w["layers.2.feed_forward.w1.weight"])
    assert torch.equal(params["layers.2.feed_forward.w13"][512:], w["layers.2.feed_forward.w3.weight"])
    assert params["norm.weight"].dtype == torch.float32


def test_loader_takes_the_reference_own_tensor_names(tmp_path):
    """A checkpoint under the reference's state-dict names (already converted: interleaved
    rows, fused wqkv; or wq, wk, wv apart, which model.py:184-189 joins as they are) gives
    the same parameters as the folder it was converted from; the names choose the layout."""
    folder = _folder(tmp_path, "B")
    arch, cfg = gfa.read_model_folder(folder)
    want = load_parameters(folder, arch.layouts(cfg), "float32", None)
    pcfg, w = plain.load_folder(folder)
    H, G, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    for split in (False, True):
        tensors = {}
        for name, t in w.items():
            if split and name.endswith("attention.wqkv.weight"):
                q, k, v = t.split([H * hd, G * hd, G * hd])
                stem = name[:-len("wqkv.weight")]
                tensors[stem + "wq.weight"], tensors[stem + "wk.weight"] = q.clone(), k.clone()
                tensors[stem + "wv.weight"] = v.clone()
            else:
                tensors[name] = t.clone()
        tensors["freqs_cis"] = torch.zeros(4, 2)                        # a buffer: ignored
        native = str(tmp_path / f"native{int(split)}")
        os.makedirs(native)
        write_safetensors(os.path.join(native, "model.safetensors"), tensors)
        with open(os.path.join(native, "config.json"), "w") as g:
            json.dump(util.TINY_B, g)
        got = load_parameters(native, arch.layouts(cfg), "float32", None)
        assert got.keys() == want.keys()
        for name in want:
            assert torch.equal(got[name], want[name]), name
        # errors are reported in the names the file uses
        del tensors["layers.1.ffn_norm.weight"]
        write_safetensors(os.path.join(native, "model.safetensors"), tensors)
        with pytest.raises(WeightsError) as e:
            load_parameters(native, arch.layouts(cfg), "float32", None)
        assert e.value.missing == ["layers.1.ffn_norm.weight"] and not e.value.unexpected


def test_loader_dtypes(tmp_path):
    folder = _folder(tmp_path, "A", dtype="bfloat16")
    arch, cfg = gfa.read_model_folder(folder)
    p = load_parameters(folder, arch.bindings(cfg), "bfloat16", None)
    assert p["layers.0.attention.wo"].dtype == torch.bfloat16          # matrices: compute type
    assert p["layers.0.ffn_norm.weight"].dtype == torch.float32         # vectors: 32-bit
    p32 = load_parameters(folder, arch.bindings(cfg), "float32", None)
    assert p32["layers.0.attention.wo"].dtype == torch.float32
    assert torch.equal(p32["layers.0.attention.wo"], p["layers.0.attention.wo"].float())


def test_tied_embeddings(tmp_path):
    folder = _folder(tmp_path, "C")
    names = SafetensorsFile(os.path.join(folder, "model.safetensors")).entries
    assert "lm_head.weight" not in names
    arch, cfg = gfa.read_model_folder(folder)
    p = load_parameters(folder, arch.bindings(cfg), "float32", None)
    assert p["output.weight"].data_ptr() == p["tok_embeddings.weight"].data_ptr()


def test_one_error_lists_everything(tmp_path):
    folder = _folder(tmp_path, "A")
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {k: f.tensor(k).clone() for k in f.entries}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(32, 64)
    tensors["model.layers.7.extra.weight"] = torch.zeros(2)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)     # ignored
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    write_safetensors(os.path.join(bad, "model.safetensors"), tensors)
    with open(os.path.join(bad, "config.json"), "w") as g:
        json.dump(util.TINY_A, g)
    arch, cfg = gfa.read_model_folder(bad)
    with pytest.raises(WeightsError) as e:
        load_parameters(bad, arch.bindings(cfg), "float32", None)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (64, 64))]
    text = str(err)
    for word in ("missing", "unexpected", "wrong shapes", "up_proj", "extra", "[32, 64]"):
        assert word in text


def test_missing_files(tmp_path):
    with pytest.raises(FileNotFoundError, match="config.json"):
        gfa.read_model_folder(str(tmp_path))
    with open(tmp_path / "config.json", "w") as g:
        json.dump(util.TINY_A, g)
    arch, cfg = gfa.read_model_folder(str(tmp_path))
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        load_parameters(str(tmp_path), arch.bindings(cfg), "float32", None)


def test_random_model_is_seeded_and_sharded_index_is_read(tmp_path):
    a = util.make_folder(tmp_path / "x", "A", seed=5)
    b = util.make_folder(tmp_path / "y", "A", seed=5)
    c = util.make_folder(tmp_path / "z", "A", seed=6)
    fa, fb, fc = (SafetensorsFile(os.path.join(f, "model.safetensors")) for f in (a, b, c))
    name = "model.layers.1.self_attn.q_proj.weight"
    assert torch.equal(fa.tensor(name), fb.tensor(name))
    assert not torch.equal(fa.tensor(name), fc.tensor(name))
    norm = fa.tensor("model.layers.0.input_layernorm.weight")
    assert abs(float(norm.mean()) - 1.0) < 0.1                  # 1 + N(0, 0.1)
    cfg = json.load(open(os.path.join(a, "config.json")))
    assert cfg["architectures"] == ["LlamaForCausalLM"] and cfg["hidden_size"] == 64
    # split into two shards with an index file
    tensors = {k: fa.tensor(k).clone() for k in fa.entries}
    keys = sorted(tensors)
    sh = str(tmp_path / "sharded")
    os.makedirs(sh)
    write_safetensors(os.path.join(sh, "m-1.safetensors"), {k: tensors[k] for k in keys[:5]})
    write_safetensors(os.path.join(sh, "m-2.safetensors"), {k: tensors[k] for k in keys[5:]})
    index = {"weight_map": {k: ("m-1.safetensors" if i < 5 else "m-2.safetensors")
                            for i, k in enumerate(keys)}}
    json.dump(index, open(os.path.join(sh, "model.safetensors.index.json"), "w"))
    json.dump(cfg, open(os.path.join(sh, "config.json"), "w"))
    arch, c2 = gfa.read_model_folder(sh)
    p1 = load_parameters(sh, arch.bindings(c2), "float32", None)
    p0 = load_parameters(a, arch.bindings(c2), "float32", None)
    assert all(torch.equal(p0[k], p1[k]) for k in p0)


def test_presets_are_found_through_the_registry():
    from gpt_fast_amd.config.registry import find_preset
    arch, cfg = find_preset("llama-3.1-8b")
    assert arch is gfa.architecture("llama") and cfg.hidden_size == 4096
    arch, cfg = find_preset("tiny-llama-b", "LlamaForCausalLM")
    assert cfg.num_key_value_heads == 2
    with pytest.raises(UnknownArchitecture, match="preset"):
        find_preset("no-such-model")
    with pytest.raises(UnknownArchitecture):
        find_preset("7B", "no-such-architecture")


def test_roles_and_inits_are_open_tables(tmp_path):
    """A parameter of a further kind - kept in float32 whatever the engine computes in,
    drawn from a law of its own - needs an entry in two tables and no change to the
    loader or to the random-weights mode."""
    from gpt_fast_amd.weights import bindings as B
    from gpt_fast_amd.weights import random_init as R
    B.register_role("toy_decay", lambda dtype: torch.float32)
    R.register_init("toy_unit_interval", lambda t, std, norm_std: torch.sigmoid(t))
    try:
        layout = B.CheckpointLayout((
            B.Binding("decay", (B.Source("blk.decay", (5, 3), "toy_unit_interval"),), role="toy_decay"),
            B.Binding("mix", (B.Source("blk.mix", (4, 4)),)),
        ))
        ck = R.random_checkpoint(layout, seed=1, dtype="bfloat16")
        assert ck["blk.decay"].min() > 0 and ck["blk.decay"].max() < 1
        write_safetensors(str(tmp_path / "model.safetensors"),
                          {"blk.decay": ck["blk.decay"].float(), "blk.mix": ck["blk.mix"]})
        params = load_parameters(str(tmp_path), layout, "bfloat16", None)
        assert params["decay"].dtype == torch.float32 and params["mix"].dtype == torch.bfloat16
        drawn = R.random_parameters(layout, 1, "bfloat16", "cpu")
        assert drawn["decay"].dtype == torch.float32
    finally:
        del B.ROLES["toy_decay"], R.INITS["toy_unit_interval"]
    with pytest.raises(ValueError, match="role"):
        B.dtype_for_role("toy_decay", torch.bfloat16)
    with pytest.raises(ValueError, match="init"):
        R.draw(B.Source("x", (2,), "toy_unit_interval"), 0, "cpu", 0.02, 0.1)


def test_text_prompts_start_with_bos(tmp_path):
    """generate.py:213-217: the BOS id goes in front.  A tokenizer.json has no BOS id of its
    own; it comes from the model's configuration."""
    from gpt_fast_amd.engine.tokenizer import Tokenizer, encode_tokens, get_tokenizer

    class Stub(Tokenizer):
        def encode(self, text):
            return [len(w) for w in text.split()]

        def bos_id(self):
            return 99

    assert encode_tokens(Stub(), "a bb ccc") == [99, 1, 2, 3]
    assert encode_tokens(Stub(), "a bb", bos=False) == [1, 2]
    tokenizers = pytest.importorskip("tokenizers")
    tk = tokenizers.Tokenizer(tokenizers.models.WordLevel({"w0": 0, "w1": 1, "w2": 2}, unk_token="w0"))
    tk.pre_tokenizer = tokenizers.pre_tokenizers.Whitespace()
    tk.save(str(tmp_path / "tokenizer.json"))
    t = get_tokenizer(str(tmp_path), bos=7, eos=8)
    assert encode_tokens(t, "w2 w1") == [7, 2, 1] and t.eos_id() == 8
    assert encode_tokens(get_tokenizer(str(tmp_path)), "w2 w1") == [2, 1]    # no id known: none added


def test_sentencepiece_model_in_a_folder(tmp_path):
    """tokenizer.py:24-39: a ``tokenizer.model`` read with sentencepiece; the model is trained
    here from a few sentences.  Encoding a text for generation puts its BOS id in front
    (generate.py:213-217) and decoding gives the text back."""
    spm = pytest.importorskip("sentencepiece")
    from gpt_fast_amd.engine.tokenizer import SentencePieceTokenizer, encode_tokens, get_tokenizer
    corpus = tmp_path / "corpus.txt"
    words = "the quick brown fox jumps over a lazy dog while seven wizards brew quiet potions".split()
    lines = [" ".join(words[(i * 3 + j) % len(words)] for j in range(7)) for i in range(200)]
    corpus.write_text("\n".join(lines) + "\n")
    spm.SentencePieceTrainer.train(input=str(corpus), model_prefix=str(tmp_path / "tokenizer"),
                                   vocab_size=60, model_type="bpe", bos_id=1, eos_id=2, unk_id=0,
                                   minloglevel=2)
    t = get_tokenizer(str(tmp_path))
    assert isinstance(t, SentencePieceTokenizer)
    assert (t.bos_id(), t.eos_id()) == (1, 2)
    ids = encode_tokens(t, "the lazy fox")
    assert ids[0] == 1 and 1 not in ids[1:] and all(0 <= i < 60 for i in ids)
    assert t.decode(ids) == "the lazy fox"
    assert encode_tokens(t, "the lazy fox", bos=False) == ids[1:]


def _write_rank_file(path, merges):
    import base64
    ranks = [bytes([b]) for b in range(256)] + [m.encode() for m in merges]
    path.write_bytes(b"".join(base64.b64encode(b) + b" " + str(r).encode() + b"\n"
                              for r, b in enumerate(ranks)))
    return len(ranks)


def test_rank_file_tokenizer_merges_by_lowest_rank(tmp_path):
    """tokenizer.py:41-95: the Llama-3 family's ``tokenizer.model`` is a list of byte strings
    with their ranks.  The reference hands it to the tiktoken package, which is not installed
    here, so parity with that package is unpinned; what is checked is the algorithm on a file
    made here: pieces by the reference's pattern, within a piece the pair of lowest rank
    first, special tokens behind the ranks in the reference's order."""
    pytest.importorskip("regex")
    from gpt_fast_amd.engine.tokenizer import RankFileTokenizer, encode_tokens, get_tokenizer
    n = _write_rank_file(tmp_path / "tokenizer.model", ["he", "ll", "hell", " w", "lo", "hello"])
    t = get_tokenizer(str(tmp_path))
    assert isinstance(t, RankFileTokenizer)
    he, ll, hell, _w, lo, hello = range(256, 262)
    assert t.encode("hello") == [hello]                   # a whole piece with a rank of its own
    # "hellow": he (256), then ll (257), then hell (258), then hello (261); w stays a byte
    assert t.encode("hellow") == [hello, ord("w")]
    # "hellx": the same merges up to hell; x stays a byte
    assert t.encode("hellx") == [hell, ord("x")]
    # "helo": he first, which leaves l, o to form lo
    assert t.encode("helo") == [he, lo]
    # "llo": ll has the lower rank, so lo is never formed
    assert t.encode("llo") == [ll, ord("o")]
    # the pattern keeps a leading space with its word: " w" + "orld"
    assert t.encode("hello world") == [hello, _w, ord("o"), ord("r"), ord("l"), ord("d")]
    assert t.encode("") == []
    assert (t.bos_id(), t.eos_id()) == (n, n + 1)
    assert t.special["<|eot_id|>"] == n + 9 and len(t.special) == 256
    ids = encode_tokens(t, "hello w\u00f6rld 123")
    assert ids[0] == n and t.decode(ids[1:]) == "hello w\u00f6rld 123"


def test_a_tokenizer_file_that_cannot_be_read_says_why(tmp_path):
    from gpt_fast_amd.engine.tokenizer import TokenizerError, get_tokenizer
    assert get_tokenizer(str(tmp_path)) is None                 # no file: no tokenizer, no error
    (tmp_path / "tokenizer.model").write_bytes(b"\x00\x01 this is neither kind of model")
    with pytest.raises(TokenizerError, match="tokenizer.model"):
        get_tokenizer(str(tmp_path))
    (tmp_path / "tokenizer.json").write_text("{ not json")
    with pytest.raises(TokenizerError, match="tokenizer.model.*tokenizer.json"):
        get_tokenizer(str(tmp_path))


def test_sizes_and_work_of_a_step_come_from_the_architecture_and_the_parts():
    """What a benchmark reports is asked of the architecture (flat sizes) and of the model's
    parts (matrix-product work of a step), not read from one configuration class's fields.
    The 8B shape's 2,048-token prompt by hand: linears, the causal triangle, one row of the
    head (model.py:136-146, 191-227)."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.parts import Runtime
    from gpt_fast_amd.parts.model import DecoderModel
    arch, cfg = gfa.find_preset("llama-3.1-8b")
    sizes = arch.describe(cfg)
    assert sizes["n_layer"] == 32 and sizes["dim"] == 4096 and sizes["n_kv_heads"] == 8
    assert sizes["intermediate_size"] == 14336 and sizes["vocab_size"] == 128256
    assert sizes["rope_scaling"].startswith("llama3 factor 8") and len(sizes) <= 12
    assert all(isinstance(v, (int, float, str)) for v in sizes.values())
    model = DecoderModel(arch.plan(cfg), Runtime(torch.bfloat16, "cpu"))
    D, H, G, hd, I, V, L, T = 4096, 32, 8, 128, 14336, 128256, 32, 2048
    linears = 2.0 * T * L * ((H + 2 * G) * hd * D + H * hd * D + 3 * I * D)
    triangle = L * 2.0 * 2.0 * H * hd * (T * (T + 1) / 2)
    assert model.step_flops([T], [0], n_want=1) == linears + triangle + 2.0 * D * V
    # a one-token step at position 100 for each of three sequences
    one = model.step_flops([1, 1, 1], [100, 100, 100], n_want=3)
    assert one == 3 * (linears / T + L * 4.0 * H * hd * 101 + 2.0 * D * V)
    raw = arch.config_dict(cfg)
    assert raw[arch.layer_count_key] == 32


def test_a_library_is_rebuilt_when_its_source_changes(tmp_path, monkeypatch):
    """The stamp beside a built library holds a hash of source, common header and flags; a
    library whose stamp does not fit is not current."""
    from gpt_fast_amd.csrc import build as b
    (tmp_path / "toy.hip").write_text("// one\n")
    (tmp_path / "common.h").write_text("// header\n")
    monkeypatch.setattr(b, "HERE", str(tmp_path))
    lib = tmp_path / "libgfa_toy.so"
    assert not b._is_current(str(lib), "toy")                       # nothing built
    lib.write_text("binary")
    assert not b._is_current(str(lib), "toy")                       # no stamp
    (tmp_path / "libgfa_toy.so.stamp").write_text(b.source_hash("toy"))
    assert b._is_current(str(lib), "toy")
    (tmp_path / "toy.hip").write_text("// two\n")
    assert not b._is_current(str(lib), "toy")                       # source edited
    (tmp_path / "libgfa_toy.so.stamp").write_text(b.source_hash("toy"))
    (tmp_path / "common.h").write_text("// header, edited\n")
    assert not b._is_current(str(lib), "toy")                       # header edited
    (tmp_path / "libgfa_toy.so.stamp").write_text(b.source_hash("toy"))
    monkeypatch.setattr(b, "FLAGS", b.FLAGS + ["-DX"])
    assert not b._is_current(str(lib), "toy")                       # flags changed


def test_plugins_named_in_the_environment_are_imported_with_the_package(tmp_path):
    """An architecture registered by a module outside the package is known to every program
    of the library (command line, trace replay) when GPT_FAST_AMD_PLUGINS names the module."""
    import subprocess
    import sys
    (tmp_path / "my_plugin.py").write_text(
        "from gpt_fast_amd.config.registry import Architecture, register_architecture\n"
        "register_architecture(Architecture(names=('PluggedIn',), read_config=dict, plan=None,\n"
        "                                   bindings=None, config_dict=dict))\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, GPT_FAST_AMD_PLUGINS="my_plugin",
               PYTHONPATH=os.pathsep.join([str(tmp_path), root, os.environ.get("PYTHONPATH", "")]))
    out = subprocess.run([sys.executable, "-c",
                          "import gpt_fast_amd as g; print('PluggedIn' in g.known_architectures())"],
                         env=env, capture_output=True, text=True, cwd=root)
    assert out.returncode == 0 and out.stdout.strip() == "True", out.stderr[-500:]
    env["GPT_FAST_AMD_PLUGINS"] = "no_such_module_anywhere"
    out = subprocess.run([sys.executable, "-c", "import gpt_fast_amd"], env=env,
                         capture_output=True, text=True, cwd=root)
    assert out.returncode != 0 and "no_such_module_anywhere" in out.stderr
