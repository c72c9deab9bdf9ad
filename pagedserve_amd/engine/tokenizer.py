"""Tokenizers for text prompts.  Token ids are the engine's primary interface."""

import os


class TokenizerError(ValueError):
    """A model folder whose tokenizer files cannot be used with its model."""


class ByteTokenizer:
    """UTF-8 bytes as tokens 0..255 and an end token 256 (src/model/tokenizer.py:1-20), for
    models whose vocabulary is exactly that."""

    vocab_size = 257

    def __init__(self, eos_token_id=256):
        self.eos_token_id = eos_token_id

    def encode(self, text):
        if not isinstance(text, str):
            raise TypeError("ByteTokenizer expects a string")
        return list(text.encode("utf-8"))

    def decode(self, token_ids):
        data = []
        for token in token_ids:
            if self.eos_token_id is not None and token == self.eos_token_id:
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
    """The folder's own tokenizer, read with the ``tokenizers`` package: ``tokenizer.json``, or
    the byte-level BPE pair ``vocab.json`` + ``merges.txt`` that GPT-2 checkpoints carry (the
    reference lets the library read them, src/model/gpt2.py:92)."""

    def __init__(self, tokenizer, eos_token_id=None):
        self._tokenizer = tokenizer
        self.eos_token_id = eos_token_id
        self.vocab_size = tokenizer.get_vocab_size()

    @classmethod
    def from_json(cls, path, eos_token_id=None):
        from tokenizers import Tokenizer

        return cls(Tokenizer.from_file(path), eos_token_id)

    @classmethod
    def from_bpe_files(cls, vocab_path, merges_path, eos_token_id=None):
        from tokenizers import Tokenizer, decoders, models, pre_tokenizers

        tokenizer = Tokenizer(models.BPE.from_file(vocab_path, merges_path))
        tokenizer.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
        tokenizer.decoder = decoders.ByteLevel()
        return cls(tokenizer, eos_token_id)

    def encode(self, text):
        return self._tokenizer.encode(text).ids

    def decode(self, token_ids):
        return self._tokenizer.decode(list(token_ids))


def load_tokenizer(folder, vocab_size, eos_token_id=None):
    """The tokenizer that belongs to a model: the folder's own files if it has any; bytes for
    the byte vocabulary of 257 entries (what the reference pairs its random model with,
    main.py:104-105); else prompts are token ids.  A vocabulary is never guessed: tokenizer
    files that do not fit the model are an error, and no other vocabulary falls back to bytes."""
    names = {name: os.path.join(folder, name) for name in ("tokenizer.json", "vocab.json", "merges.txt")
             if folder and os.path.isfile(os.path.join(folder, name))}
    tokenizer = None
    if "tokenizer.json" in names:
        tokenizer = FileTokenizer.from_json(names["tokenizer.json"], eos_token_id)
    elif "vocab.json" in names and "merges.txt" in names:
        tokenizer = FileTokenizer.from_bpe_files(names["vocab.json"], names["merges.txt"], eos_token_id)
    elif names:
        raise TokenizerError(f"{folder!r} holds {', '.join(sorted(names))} only: a byte-level BPE "
                             "tokenizer needs vocab.json and merges.txt (or one tokenizer.json)")
    if tokenizer is not None:
        if tokenizer.vocab_size > vocab_size:
            raise TokenizerError(f"the tokenizer of {folder!r} has {tokenizer.vocab_size} tokens, "
                                 f"the model's vocabulary only {vocab_size}")
        return tokenizer
    if vocab_size == ByteTokenizer.vocab_size:
        return ByteTokenizer(eos_token_id)
    return IdTokenizer(eos_token_id)
