"""Command line in the manner of the reference's generate.py (its flags at
generate.py:450-463, its driver at :272-437).

    python -m gpt_fast_amd --checkpoint_path MODEL_FOLDER --prompt "Hello, my name is"
    python -m gpt_fast_amd --random llama-3.1-8b --prompt 128 --batch_size 8

``--random`` takes a preset's name (of whichever registered architecture knows it, or of
``--architecture``) or the path of a config.json.  ``--checkpoint_path`` names a model *folder* (config.json + safetensors; the reference
takes a converted model.pth whose folder name selects the configuration,
generate.py:222).  ``--prompt`` is text, or an integer N for a synthetic prompt of N
random token ids below min(1024, vocabulary) as in generate.py:325-327.  Flags of the
reference that have no meaning here (--compile, --compile_prefill: the kernels are
compiled ahead of time) are accepted and ignored; those of features outside this
library (--speculate_k, --draft_checkpoint_path) are refused.  ``--interactive`` asks for
every sample's prompt and writes its text as it is drawn (generate.py:356-377).
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path
from typing import List, Optional, Union

import torch

from ..cache.store import pages_for
from ..config.registry import architecture_of, find_preset, read_model_folder
from ..ops.kernels import PAGE
from ..sampling import SamplingParams
from .generate import generate
from .step import Engine
from .tokenizer import TokenizerError, encode_tokens, get_tokenizer


B_INST, E_INST = "[INST]", "[/INST]"          # generate.py:270
INTERACTIVE_POSITIONS = 350                   # generate.py:161


def _int_or_str(x):
    try:
        return int(x)
    except ValueError:
        return x


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="gpt_fast_amd", description="Generate with a Llama model "
                                "on an MI355X.")
    p.add_argument("--prompt", type=_int_or_str, default="Hello, my name is",
                   help="Input prompt. If it's an integer, will instead generate a synthetic prompt.")
    p.add_argument("--prompt_ids", type=str, default=None,
                   help="Comma-separated token ids to use as the prompt instead of --prompt.")
    p.add_argument("--interactive", action="store_true", help="Whether to launch in interactive mode")
    p.add_argument("--num_samples", type=int, default=5, help="Number of samples.")
    p.add_argument("--max_new_tokens", type=int, default=200, help="Maximum number of new tokens.")
    p.add_argument("--batch_size", type=int, default=1, help="Batch size to benchmark with")
    p.add_argument("--top_k", type=int, default=200, help="Top-k for sampling.")
    p.add_argument("--temperature", type=float, default=0.8, help="Temperature for sampling.")
    p.add_argument("--checkpoint_path", type=Path, default=None,
                   help="Model folder (config.json and safetensors files).")
    p.add_argument("--random", type=str, default=None, metavar="PRESET",
                   help="Use seeded random weights of a named configuration (or of a "
                        "config.json file) instead of a folder.")
    p.add_argument("--architecture", type=str, default=None,
                   help="Architecture whose preset --random names (default: the one that "
                        "knows the name).")
    p.add_argument("--seed", type=int, default=1234, help="Seed of sampling and of --random.")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--max_seq_length", type=int, default=None,
                   help="Cache positions per sequence (default: prompt + new tokens).")
    p.add_argument("--compile", action="store_true", help="Accepted for compatibility; no effect.")
    p.add_argument("--compile_prefill", action="store_true",
                   help="Accepted for compatibility; no effect.")
    p.add_argument("--profile", type=Path, default=None, help="Profile path.")
    p.add_argument("--speculate_k", type=int, default=None, help="(not available)")
    p.add_argument("--draft_checkpoint_path", type=Path, default=None, help="(not available)")
    p.add_argument("--device", type=str, default="cuda", help="Device to use")
    return p


def main(prompt: Union[int, str, List[int]] = "Hello, my name is", num_samples: int = 5,
         max_new_tokens: int = 100, batch_size: int = 1, top_k: Optional[int] = 200,
         temperature: float = 0.8, checkpoint_path: Optional[Path] = None,
         random: Optional[str] = None, seed: int = 1234, dtype: str = "bfloat16",
         max_seq_length: Optional[int] = None, profile: Optional[Path] = None,
         device: str = "cuda", architecture_name: Optional[str] = None, out=print,
         interactive: bool = False, input_fn=input, stream=None) -> dict:
    """Generates samples and reports throughput the way the reference's ``main`` does
    (generate.py:272-437).  Returns the aggregate numbers it printed.

    ``interactive``: every sample asks for its prompt (``input_fn``) and its text is written
    to ``stream`` as it is drawn, four tokens at a time (generate.py:356-377); a folder whose
    path contains "chat" gets the prompt wrapped in [INST] .. [/INST] (generate.py:298, 359);
    prompt and new tokens share ``max_seq_length`` positions, 350 unless given
    (generate.py:160-161)."""
    if (checkpoint_path is None) == (random is None):
        raise SystemExit("give either --checkpoint_path MODEL_FOLDER or --random PRESET")
    device = "cuda:0" if device == "cuda" else device
    out(f"Using device={device}")

    # the model class and its configuration: by the folder's config.json, or by the preset's
    # name among the registered architectures (or a config.json file given as the preset)
    if checkpoint_path is not None:
        arch, config = read_model_folder(str(checkpoint_path))
    elif os.path.isfile(random):
        with open(random) as f:
            raw = json.load(f)
        arch = architecture_of(raw)
        config = arch.read_config(raw)
    else:
        arch, config = find_preset(random, architecture_name)

    tokenizer = None
    if isinstance(prompt, list):
        encoded = [int(t) for t in prompt]
    elif isinstance(prompt, int):
        encoded = None                       # synthetic, needs the vocabulary size
    else:
        eos = getattr(config, "eos_token_id", None) or ()
        try:
            tokenizer = get_tokenizer(str(checkpoint_path), bos=getattr(config, "bos_token_id", None),
                                      eos=eos[0] if eos else None) if checkpoint_path else None
        except TokenizerError as e:
            raise SystemExit(str(e))
        if tokenizer is None:
            raise SystemExit("a text prompt needs a tokenizer.model or tokenizer.json in the "
                             "model folder (and sentencepiece or tokenizers); use an integer "
                             "--prompt for a synthetic prompt, or --prompt_ids")
        encoded = encode_tokens(tokenizer, prompt, bos=True)          # generate.py:213-217
    prompt_length = prompt if encoded is None else len(encoded)
    if prompt_length < 1:
        raise SystemExit("the prompt needs at least one token")
    is_chat = checkpoint_path is not None and "chat" in str(checkpoint_path)
    if interactive:
        if tokenizer is None:
            raise SystemExit("--interactive needs a text prompt and a model folder with a tokenizer")
        if stream is None:
            stream = sys.stdout
        max_seq_length = max_seq_length or INTERACTIVE_POSITIONS
    per_seq = max_seq_length or (prompt_length + max_new_tokens)
    per_seq = pages_for(per_seq) * PAGE                # the cache is handed out in whole pages
    most = getattr(arch.plan(config), "max_positions", None)
    if interactive and most is not None:
        per_seq = min(per_seq, most)                   # the model's own positions bound a dialogue
    if interactive:
        max_new_tokens = max(1, min(max_new_tokens, per_seq - prompt_length))
    if prompt_length + max_new_tokens > per_seq:
        raise SystemExit(f"prompt ({prompt_length}) + max_new_tokens ({max_new_tokens}) exceed "
                         f"--max_seq_length {per_seq}")

    out("Loading model ...")
    t0 = time.time()
    cache_args = dict(max_tokens=per_seq * batch_size, max_sequences=batch_size)
    if random is not None:
        engine = Engine.from_random(arch.names[0], config, seed, dtype=dtype, device=device,
                                    **cache_args)
    else:
        engine = Engine.from_folder(str(checkpoint_path), dtype=dtype, device=device, **cache_args)
    torch.cuda.synchronize()
    out(f"Time to load model: {time.time() - t0:.02f} seconds")

    if encoded is None:
        g = torch.Generator().manual_seed(seed)
        hi = min(1024, engine.vocab_size)
        encoded = torch.randint(0, hi, (prompt,), generator=g).tolist()
    model_size = engine.model.parameter_bytes()
    n_params = engine.model.parameter_count()
    tokens_per_sec = []
    result = None
    for i in range(-1, num_samples):                       # sample -1 warms up, generate.py:352
        torch.cuda.synchronize()
        new_tokens = max_new_tokens
        callback = None
        if interactive and i >= 0:
            text = input_fn("What is your prompt? ")
            if is_chat:
                text = f"{B_INST} {text.strip()} {E_INST}"
            encoded = encode_tokens(tokenizer, text, bos=True)
            if len(encoded) >= per_seq:
                out(f"The prompt has {len(encoded)} tokens; {per_seq} positions are there for "
                    f"prompt and answer (--max_seq_length)")
                continue
            new_tokens = min(max_new_tokens, per_seq - len(encoded))
            callback = _streamer(tokenizer, stream, engine.model.plan.stop_tokens)
        prof = None
        if profile is not None and i == num_samples - 1:      # the last sample, generate.py:380-385
            prof = torch.profiler.profile()
            prof.__enter__()
        t0 = time.perf_counter()
        result = generate(engine, [encoded] * batch_size, new_tokens,
                          temperature=temperature, top_k=top_k, seed=seed + max(i, 0),
                          callback=callback)
        torch.cuda.synchronize()
        t = time.perf_counter() - t0
        if callback is not None:
            callback.flush()
        if prof is not None:
            prof.__exit__(None, None, None)
            prof.export_chrome_trace(f"{profile}.json")
        if i == -1:
            out(f"Warm-up time: {t:.2f} seconds")
            continue
        if batch_size > 1:
            out("Only displaying the first generation of the batch")
        seq = encoded + result.tokens[0]
        if interactive:
            out("")                                       # the text has been streamed, generate.py:404-407
        else:
            out(tokenizer.decode(seq) if tokenizer is not None else " ".join(map(str, seq)))
        generated = len(result.tokens[0])
        tps = generated / t
        tokens_per_sec.append(tps)
        out(f"Time for inference {i + 1}: {t:.02f} sec total, {tps:.02f} tokens/sec")
        out(f"Bandwidth achieved: {model_size * tps / 1e9:.02f} GB/s")
        # generate.py:421-424: every token of every sequence, prompt included, per second
        total_tokens_sec = batch_size * len(seq) / t
        out(f"FLOPS achieved: {n_params * total_tokens_sec * 2 / 1e12:.02f} TF/s")
        st = result.stats
        if st.get("decode_steps"):
            out(f"Decode: {st['decode_steps'] * batch_size / st['decode_seconds']:.02f} tokens/sec "
                f"over the batch; prefill {st['prefill_seconds'] * 1e3:.1f} ms")
        out("")
    out("==========")
    out(f"Batch Size: {batch_size}")
    out(f"Prompt Length: {prompt_length}")
    out(f"Generated tokens: {max_new_tokens}")
    mean = sum(tokens_per_sec) / max(len(tokens_per_sec), 1)
    out(f"Average tokens/sec: {mean:.2f}")
    out(f"Memory used: {torch.cuda.max_memory_reserved() / 1e9:.02f} GB")
    return {"tokens_per_sec": mean, "result": result}


class _streamer:
    """Writes a request's text as its tokens are drawn, four at a time (generate.py:362-377).
    A token is decoded behind a token of known text and that text is cut off again, so that
    a tokenizer that drops the space in front of a first word keeps it here (the reference
    does this with the id of '.')."""

    def __init__(self, tokenizer, stream, stop_tokens=(), every: int = 4):
        self.tokenizer, self.stream, self.every = tokenizer, stream, every
        # what ends a request: the ids generation stops on, and the tokenizer's own end id
        self.stop = set(int(t) for t in stop_tokens or ())
        if tokenizer.eos_id() is not None:
            self.stop.add(tokenizer.eos_id())
        lead = tokenizer.encode(".")
        self.lead = lead[:1]
        self.cut = len(tokenizer.decode(self.lead)) if self.lead else 0
        self.buffer: List[str] = []
        self.done = False

    def __call__(self, rows, tokens) -> None:
        if self.done or 0 not in rows:
            return
        token = tokens[rows.index(0)]
        self.buffer.append(self.tokenizer.decode(self.lead + [token])[self.cut:])
        if token in self.stop:
            self.done = True
        if len(self.buffer) == self.every or self.done:
            self.flush()

    def flush(self) -> None:
        if self.buffer:
            self.stream.write("".join(self.buffer))
            self.stream.flush()
            self.buffer.clear()


def cli(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.speculate_k is not None or args.draft_checkpoint_path is not None:
        raise SystemExit("speculative decoding is not part of this library")
    prompt = args.prompt
    if args.prompt_ids:
        prompt = [int(t) for t in args.prompt_ids.split(",")]
    main(prompt, args.num_samples, args.max_new_tokens, args.batch_size, args.top_k,
         args.temperature, args.checkpoint_path, args.random, args.seed, args.dtype,
         args.max_seq_length, args.profile, args.device, args.architecture,
         interactive=args.interactive)
    return 0
