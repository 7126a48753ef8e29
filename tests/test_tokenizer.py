"""The command line's tokenizer (CPU); behaviour of src/io/tokenizer.cpp:80-182."""
import base64

import pytest

from photon_infer_amd import PhotonError
from photon_infer_amd.tokenizer import TikTokenizer


def write_vocab(path, tokens):
    path.write_text("".join(f"{base64.b64encode(t).decode()} {i}\n" for i, t in enumerate(tokens)))


def test_greedy_longest_match_and_byte_fallback(tmp_path):
    toks = [b"a", b"b", b"ab", b"abc", b" ", b"hello", b" world", b"\xc3", b"\xa9"]
    write_vocab(tmp_path / "v.model", toks)
    t = TikTokenizer.load(str(tmp_path / "v.model"))
    assert t.vocab_size() == len(toks)
    assert t.encode("abcab") == [3, 2]                # the longest match first, not merges
    assert t.encode("hello world") == [5, 6]
    assert t.encode("aXb") == [0, 1]                  # an unknown byte is skipped
    assert t.encode("é") == [7, 8]                    # bytes, not characters
    assert t.decode([5, 6]) == "hello world" and t.decode_token(3) == "abc"
    assert t.decode([7, 8]) == "é"


def test_special_tokens_and_errors(tmp_path):
    write_vocab(tmp_path / "v.model", [b"x"])
    t = TikTokenizer.load(str(tmp_path / "v.model"))
    assert (t.bos_id(), t.eos_id()) == (128000, 128001)
    assert t.decode_token(128000) == "<|begin_of_text|>" and t.decode_token(128001) == "<|end_of_text|>"
    assert t.decode_token(128010) == "<|reserved_special_token_10|>" and t.decode_token(555) == ""
    with pytest.raises(PhotonError, match="not found"):
        TikTokenizer.load(str(tmp_path / "none"))
    (tmp_path / "empty").write_text("\n")
    with pytest.raises(PhotonError, match="Empty"):
        TikTokenizer.load(str(tmp_path / "empty"))
