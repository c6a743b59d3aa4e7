"""Text in, ids out, for the command line only; the library's contract is ids.

The reference wraps sentencepiece for ``tokenizer.model`` files and tiktoken for the
Llama-3 family (tokenizer.py:24-112).  Here a model folder's ``tokenizer.model`` is read
with sentencepiece and a ``tokenizer.json`` with the ``tokenizers`` package, whichever
file and package are present; BOS/EOS ids come from the tokenizer, else from the model's
configuration.
"""
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


def get_tokenizer(folder: str, bos: Optional[int] = None, eos: Optional[int] = None):
    """The folder's tokenizer, or None if it has none that an installed package reads."""
    model = os.path.join(folder, "tokenizer.model")
    if os.path.isfile(model):
        try:
            return SentencePieceTokenizer(model)
        except Exception:
            pass
    js = os.path.join(folder, "tokenizer.json")
    if os.path.isfile(js):
        try:
            return JsonTokenizer(js, bos, eos)
        except Exception:
            pass
    return None


def encode_tokens(tokenizer: Tokenizer, text: str, bos: bool = True) -> List[int]:
    """generate.py:213-217: the text's ids with the BOS id in front."""
    ids = tokenizer.encode(text)
    if bos and tokenizer.bos_id() is not None:
        ids = [tokenizer.bos_id()] + ids
    return ids
