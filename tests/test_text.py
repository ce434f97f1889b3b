"""The vocabulary tokenizer and the chat format against the reference's rules
(src/tokenizer.cc, src/async_engine.cc:82-106).  The reference ships no vocabulary and no
encoded vectors; what pins the byte alphabet is its own comment (space -> U+0120,
src/tokenizer.cc:136-137) and the rule it states, what pins the matching are hand-made
vocabularies where a shorter or a later match would give other ids."""
import threading

import pytest

import configs
import plain_qwen3
import reference_ops
from lucciola_amd.text.vocab_tokenizer import ChatFormat, VocabTokenizer, byte_alphabet


def byte_vocab(extra=()):
    """Every single byte as a token (ids 0..255), then the extra tokens (given as text)."""
    alphabet = byte_alphabet()
    vocab = {alphabet[b]: b for b in range(256)}
    for text in extra:
        vocab["".join(alphabet[b] for b in text.encode("utf-8"))] = len(vocab)
    return vocab


def test_byte_alphabet():
    a = byte_alphabet()
    assert len(set(a)) == 256
    assert a[0x20] == "Ġ" and a[0x0A] == "Ċ"          # the well-known pair
    assert a[ord("!")] == "!" and a[ord("~")] == "~" and a[0xA1] == "¡" and a[0xFF] == "ÿ"
    assert a[0x00] == "Ā" and a[0x7F] == chr(256 + 33) and a[0xAD] == chr(256 + 67)
    assert sorted(ord(c) for c in a if ord(c) >= 256) == list(range(256, 256 + 68))


def test_longest_match_from_the_front():
    tok = VocabTokenizer(byte_vocab(["ab", "abc", "bcd", "cab"]))
    ids = {t: tok.token_to_id["".join(byte_alphabet()[b] for b in t.encode())] for t in ("ab", "abc", "bcd", "cab")}
    # "abcab": the longest at the front is "abc" (not "ab" + "cab"), then "ab"
    assert tok.encode("abcab") == [ids["abc"], ids["ab"]]
    # greedy, not best: "abcd" is "abc" + "d" although "a" + "bcd" has as many tokens
    assert tok.encode("abcd") == [ids["abc"], ord("d")]
    assert tok.encode("") == []


def test_text_round_trip_and_bytes_outside_ascii():
    tok = VocabTokenizer(byte_vocab(["é", " the", "日本"]))
    text = "Café in the 日本語\n\ttab \U0001F600"
    ids = tok.encode(text)
    assert tok.decode(ids) == text
    assert tok.token_to_id["Ġthe"] in ids                 # " the" as one token
    assert len(ids) < len(text.encode("utf-8"))


def test_a_character_without_an_entry_is_dropped():
    alphabet = byte_alphabet()
    vocab = {alphabet[ord("a")]: 0, alphabet[ord("b")]: 1}
    tok = VocabTokenizer(vocab)
    assert tok.encode("a?b b") == [0, 1, 1]
    assert tok.decode([0, 7, -1, 1]) == "ab"                      # ids outside the vocabulary are empty


def test_a_token_outside_the_alphabet_stands_for_itself():
    tok = VocabTokenizer({"<|x|>": 0, "日": 1, "a": 2})
    assert tok.decode([0, 2]) == "<|x|>a"
    assert tok.token_bytes(1) == "日".encode("utf-8")


def test_stream_joins_a_character_spread_over_tokens():
    tok = VocabTokenizer(byte_vocab())
    raw = "日a".encode("utf-8")                              # three bytes, then one
    stream = tok.stream()
    pieces = [stream.feed(b, last=(i == len(raw) - 1)) for i, b in enumerate(raw)]
    assert pieces == ["", "", "日", "a"]
    cut = tok.stream()
    assert cut.feed(raw[0]) == "" and cut.feed(raw[1], last=True) == "�"


def test_chat_format_layout():
    tok = VocabTokenizer(byte_vocab(["system\n", "user\n", "assistant\n"]))
    fmt = ChatFormat(start_id=900, end_id=901, enter_id=902, system="S")
    ids = fmt.prompt(tok, "hi")
    sys_id = tok.token_to_id["systemĊ"]
    usr_id = tok.token_to_id["userĊ"]
    ast_id = tok.token_to_id["assistantĊ"]
    assert ids == [900, sys_id, ord("S"), 901, 902, 900, usr_id, ord("h"), ord("i"), 901, 902, 900, ast_id]
    ref = ChatFormat()                                           # the reference's literals
    assert (ref.start_id, ref.end_id, ref.enter_id) == (151644, 151645, 1699)
    assert ref.system == "You are a helpful assistant."


def test_async_engine_takes_text(monkeypatch):
    """A text prompt through AsyncEngine: encoded inside the chat format, generated greedily,
    and handed to the callback as text, piece by piece."""
    from test_engine_host import host_engine
    from helpers import random_weights
    from lucciola_amd.engine.async_engine import AsyncEngine
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.3)
    V = cfg["vocab_size"]
    alphabet = byte_alphabet()
    # a vocabulary as large as the model's: single printable bytes first, then pairs
    printable = [chr(c) for c in range(0x20, 0x7F)] + ["\n"]
    entries = printable + [x + y for x in "abcdefgh" for y in "abcdefgh"]
    vocab = {"".join(alphabet[b] for b in e.encode()): i for i, e in enumerate(entries[:V])}
    tok = VocabTokenizer(vocab)
    fmt = ChatFormat(start_id=V - 1, end_id=V - 2, enter_id=V - 3, system="be brief")
    engine = host_engine(cfg, weights, page, 64, max_tokens_per_step=16)
    front = AsyncEngine("", engine=engine, tokenizer=tok, chat_format=fmt)
    try:
        done = threading.Event()
        pieces = []

        def on_text(text, finished):
            assert isinstance(text, str)
            pieces.append(text)
            if finished:
                done.set()
        front.generate_async("ab cd", 8, on_text)
        assert done.wait(60)
    finally:
        front.stop()
    prompt = fmt.prompt(tok, "ab cd")
    want = plain_qwen3.greedy(cfg, weights, prompt, 8)
    for i, t in enumerate(want):
        if t in engine.eos_token_ids:
            want = want[:i + 1]
            break
    assert len(pieces) == len(want) and "".join(pieces) == tok.decode(want)
    with pytest.raises(ValueError):
        AsyncEngine("", engine=engine).generate_async("text without a vocabulary", 1, lambda t, f: None)
