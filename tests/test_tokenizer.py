"""Which tokenizer a model folder gets, and that a vocabulary is never guessed."""

import json

import pytest

from pagedserve_amd.engine.tokenizer import (ByteTokenizer, FileTokenizer, IdTokenizer,
                                             TokenizerError, load_tokenizer)

VOCAB = {"h": 0, "e": 1, "l": 2, "o": 3, "Ġ": 4, "he": 5, "ll": 6, "hell": 7, "hello": 8, "Ġhello": 9}
MERGES = ["h e", "l l", "he ll", "hell o", "Ġ hello"]


def _bpe_folder(tmp_path, vocab=True, merges=True):
    if vocab:
        (tmp_path / "vocab.json").write_text(json.dumps(VOCAB))
    if merges:
        (tmp_path / "merges.txt").write_text("#version: 0.2\n" + "\n".join(MERGES) + "\n")
    return str(tmp_path)


def test_byte_level_bpe_files_are_read(tmp_path):
    tokenizer = load_tokenizer(_bpe_folder(tmp_path), vocab_size=16, eos_token_id=3)
    assert isinstance(tokenizer, FileTokenizer) and tokenizer.eos_token_id == 3
    assert tokenizer.encode("hello hello") == [8, 9]
    assert tokenizer.encode("hell") == [7]
    assert tokenizer.decode([8, 9, 4, 5]) == "hello hello he"


def test_half_a_tokenizer_and_a_tokenizer_too_large_are_refused(tmp_path):
    with pytest.raises(TokenizerError, match="vocab.json and merges.txt"):
        load_tokenizer(_bpe_folder(tmp_path, merges=False), 50257)
    (tmp_path / "merges.txt").write_text("#version: 0.2\n" + "\n".join(MERGES) + "\n")
    with pytest.raises(TokenizerError, match="10 tokens"):
        load_tokenizer(str(tmp_path), vocab_size=9)


def test_bytes_only_for_the_byte_vocabulary(tmp_path):
    folder = str(tmp_path)
    tokenizer = load_tokenizer(folder, 257, 256)
    assert isinstance(tokenizer, ByteTokenizer) and tokenizer.eos_token_id == 256
    assert tokenizer.decode(tokenizer.encode("påge") + [256, 65]) == "påge"
    # no end token: token 256 is no byte and is left out, what follows is kept
    assert load_tokenizer(folder, 257, None).decode([65, 256, 66]) == "AB"
    # any other vocabulary has no text form of its own: prompts are ids, never bytes
    for vocab in (256, 512, 50257):
        tokenizer = load_tokenizer(folder, vocab, None)
        assert isinstance(tokenizer, IdTokenizer) and tokenizer.eos_token_id is None
        assert tokenizer.encode("5 17 3") == [5, 17, 3] and tokenizer.decode([1, 2]) == "1 2"
        with pytest.raises(ValueError, match="token ids"):
            tokenizer.encode("Paged attention")
