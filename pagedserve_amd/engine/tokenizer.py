"""Tokenizers for text prompts.  Token ids are the engine's primary interface."""

import os


class ByteTokenizer:
    """UTF-8 bytes as tokens 0..255 and an end token 256 (src/model/tokenizer.py:1-20)."""

    eos_token_id = 256
    vocab_size = 257

    def encode(self, text):
        if not isinstance(text, str):
            raise TypeError("ByteTokenizer expects a string")
        return list(text.encode("utf-8"))

    def decode(self, token_ids):
        data = []
        for token in token_ids:
            if token == self.eos_token_id:
                break
            if 0 <= token < 256:
                data.append(token)
        return bytes(data).decode("utf-8", errors="replace")


class IdTokenizer:
    """Prompts are space-separated integers; output likewise.  For vocabularies that
    have no text form (random models smaller than a byte tokenizer needs)."""

    def __init__(self, eos_token_id=None):
        self.eos_token_id = eos_token_id

    def encode(self, text):
        try:
            return [int(piece) for piece in text.split()]
        except ValueError:
            raise ValueError("this model has no text tokenizer; give space-separated "
                             "token ids") from None

    def decode(self, token_ids):
        return " ".join(str(token) for token in token_ids)


class FileTokenizer:
    """The folder's own ``tokenizer.json``, read with the ``tokenizers`` package."""

    def __init__(self, path, eos_token_id=None):
        from tokenizers import Tokenizer

        self._tokenizer = Tokenizer.from_file(path)
        self.eos_token_id = eos_token_id

    def encode(self, text):
        return self._tokenizer.encode(text).ids

    def decode(self, token_ids):
        return self._tokenizer.decode(list(token_ids))


def load_tokenizer(folder, vocab_size, eos_token_id=None):
    """``tokenizer.json`` if the folder has one, else bytes if the vocabulary is large
    enough (as the reference pairs its random model with, main.py:104-105), else ids."""
    path = os.path.join(folder, "tokenizer.json") if folder else None
    if path and os.path.isfile(path):
        return FileTokenizer(path, eos_token_id)
    if vocab_size >= ByteTokenizer.vocab_size:
        return ByteTokenizer()
    return IdTokenizer(eos_token_id)
