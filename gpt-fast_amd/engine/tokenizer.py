"""Text in, ids out, for the command line only; the library's contract is ids.

The reference wraps sentencepiece for ``tokenizer.model`` files and tiktoken for the
Llama-3 family, whose ``tokenizer.model`` is a list of byte strings with their ranks
(tokenizer.py:24-112).  Here a model folder's ``tokenizer.model`` is read with sentencepiece,
or - if it is such a rank file - by the byte-pair encoder of this module (the reference picks
by the model's name, tokenizer.py:109; here the file's first line tells); a ``tokenizer.json``
is read with the ``tokenizers`` package.  BOS/EOS ids come from the tokenizer, else from the
model's configuration.  A file that is there but cannot be read is an error that says why.
"""
import base64
import os
from typing import List, Optional


class Tokenizer:
    def encode(self, text: str) -> List[int]:
        raise NotImplementedError

    def decode(self, ids: List[int]) -> str:
        raise NotImplementedError

    def bos_id(self) -> Optional[int]:
        return None

    def eos_id(self) -> Optional[int]:
        return None


class SentencePieceTokenizer(Tokenizer):
    def __init__(self, path: str):
        import sentencepiece as spm
        self.sp = spm.SentencePieceProcessor(model_file=path)

    def encode(self, text):
        return list(self.sp.EncodeAsIds(text))

    def decode(self, ids):
        return self.sp.DecodeIds(list(ids))

    def bos_id(self):
        i = self.sp.bos_id()
        return i if i >= 0 else None

    def eos_id(self):
        i = self.sp.eos_id()
        return i if i >= 0 else None


class JsonTokenizer(Tokenizer):
    def __init__(self, path: str, bos: Optional[int], eos: Optional[int]):
        from tokenizers import Tokenizer as _T
        self.tk = _T.from_file(path)
        self._bos, self._eos = bos, eos

    def encode(self, text):
        return list(self.tk.encode(text, add_special_tokens=False).ids)

    def decode(self, ids):
        return self.tk.decode(list(ids))

    def bos_id(self):
        return self._bos

    def eos_id(self):
        return self._eos


class RankFileTokenizer(Tokenizer):
    """Byte-pair encoding from a rank file: every line holds a byte string in base64 and its
    rank, which is also its id (the format of the Llama-3 family's ``tokenizer.model``,
    tokenizer.py:53-54).  The text is cut into pieces by the reference's pattern
    (tokenizer.py:50); within a piece, the adjacent pair of parts whose concatenation has
    the lowest rank is merged until no pair has a rank.  The special tokens follow the
    ranks in the reference's order (tokenizer.py:56-72): BOS is the first, EOS the second."""

    PIECES = (r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}{1,3}|"
              r" ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+")
    RESERVED = 256

    def __init__(self, path: str):
        import regex                       # \p{L} classes: not in the standard library's re
        self.ranks = read_rank_file(path)
        if not self.ranks:
            raise ValueError("the rank file is empty")
        self.pattern = regex.compile(self.PIECES)
        n = len(self.ranks)
        names = ["<|begin_of_text|>", "<|end_of_text|>", "<|reserved_special_token_0|>",
                 "<|reserved_special_token_1|>", "<|reserved_special_token_2|>",
                 "<|reserved_special_token_3|>", "<|start_header_id|>", "<|end_header_id|>",
                 "<|reserved_special_token_4|>", "<|eot_id|>"]
        names += [f"<|reserved_special_token_{i}|>" for i in range(5, self.RESERVED - 5)]
        self.special = {name: n + i for i, name in enumerate(names)}
        self.by_id = {r: b for b, r in self.ranks.items()}
        self.by_id.update({i: name.encode("utf-8") for name, i in self.special.items()})

    def _piece(self, piece: bytes) -> List[int]:
        if piece in self.ranks:
            return [self.ranks[piece]]
        parts = [piece[i:i + 1] for i in range(len(piece))]
        while len(parts) > 1:
            best, at = None, -1
            for i in range(len(parts) - 1):
                r = self.ranks.get(parts[i] + parts[i + 1])
                if r is not None and (best is None or r < best):
                    best, at = r, i
            if best is None:
                break
            parts[at:at + 2] = [parts[at] + parts[at + 1]]
        missing = [p for p in parts if p not in self.ranks]
        if missing:
            raise ValueError(f"the rank file has no entry for the byte string {missing[0]!r}")
        return [self.ranks[p] for p in parts]

    def encode(self, text):
        ids: List[int] = []
        for piece in self.pattern.findall(text):
            ids += self._piece(piece.encode("utf-8"))
        return ids

    def decode(self, ids):
        return b"".join(self.by_id[int(i)] for i in ids).decode("utf-8", errors="replace")

    def bos_id(self):
        return self.special["<|begin_of_text|>"]

    def eos_id(self):
        return self.special["<|end_of_text|>"]


def read_rank_file(path: str):
    """{byte string: rank} of a rank file; raises ValueError if the file is not one."""
    ranks = {}
    with open(path, "rb") as f:
        for n, line in enumerate(f):
            if not line.strip():
                continue
            fields = line.split()
            if len(fields) != 2:
                raise ValueError(f"line {n + 1} is not '<base64> <rank>'")
            ranks[base64.b64decode(fields[0], validate=True)] = int(fields[1])
    return ranks


def _is_rank_file(path: str) -> bool:
    """The first line reads '<base64> <integer>' (a sentencepiece model is a binary record)."""
    with open(path, "rb") as f:
        first = f.readline(4096).split()
    try:
        base64.b64decode(first[0], validate=True)
        int(first[1])
        return len(first) == 2
    except (IndexError, ValueError):
        return False


class TokenizerError(RuntimeError):
    pass


def get_tokenizer(folder: str, bos: Optional[int] = None, eos: Optional[int] = None):
    """The folder's tokenizer: ``tokenizer.model`` first, else ``tokenizer.json``; None if the
    folder has neither.  If a file is there and none can be read (a missing package, a file
    of another kind), :class:`TokenizerError` says what each attempt failed with."""
    problems = []
    model = os.path.join(folder, "tokenizer.model")
    if os.path.isfile(model):
        try:
            if _is_rank_file(model):
                return RankFileTokenizer(model)
            return SentencePieceTokenizer(model)
        except Exception as e:
            problems.append(f"tokenizer.model: {type(e).__name__}: {e}")
    js = os.path.join(folder, "tokenizer.json")
    if os.path.isfile(js):
        try:
            return JsonTokenizer(js, bos, eos)
        except Exception as e:
            problems.append(f"tokenizer.json: {type(e).__name__}: {e}")
    if problems:
        raise TokenizerError(f"{folder}: no tokenizer could be read - " + "; ".join(problems))
    return None


def encode_tokens(tokenizer: Tokenizer, text: str, bos: bool = True) -> List[int]:
    """generate.py:213-217: the text's ids with the BOS id in front."""
    ids = tokenizer.encode(text)
    if bos and tokenizer.bos_id() is not None:
        ids = [tokenizer.bos_id()] + ids
    return ids
