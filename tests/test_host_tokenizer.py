"""The host tokenizer: the reference's own known-answer tests (crates/neura-tokenizer/tests/tokenizer.rs) run against the
C++ mirror, and the Qwen2 split rule checked against the published pattern run by the `regex` module."""
import random

import pytest

from gguf_fixture import build as build_gguf
from neura_amd import host

QWEN2_PATTERN = (r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+")


def archive(tokens, kinds, merges, model="gpt2"):
    data, _, _ = build_gguf(32, [("tokenizer.ggml.model", "string", model), ("tokenizer.ggml.tokens", "array", ("string", list(tokens))),
                                 ("tokenizer.ggml.token_type", "array", ("u32", list(kinds))),
                                 ("tokenizer.ggml.merges", "array", ("string", list(merges)))], [])
    return host.Gguf.decode(data)


def refuses(action, sentence=None):
    with pytest.raises(host.Panic) as raised:
        action()
    if sentence:
        assert sentence in str(raised.value), str(raised.value)


def test_a_byte_reads_back_as_the_token_it_spells():
    # tokenizer.rs:58-74
    source = archive(["A", "!", "Ġ", "Ċ", "ġ"], [1] * 5, [])
    tokenizer = host.Tokenizer(source, "per_character")
    ids = tokenizer.encode("A! \n\x7f")
    assert ids == [0, 1, 2, 3, 4]
    assert b"".join(tokenizer.piece(id) for id in ids) == "A! \n\x7f".encode()


def test_a_piece_of_several_bytes_rounds_through_the_alphabet():
    # tokenizer.rs:76-86
    source = archive(["Ã", "©", "Ã©"], [1, 1, 1], ["Ã ©"])
    tokenizer = host.Tokenizer(source, "whole")
    assert tokenizer.encode("é") == [2]
    assert tokenizer.piece(2) == "é".encode()


def test_a_special_token_stands_apart_from_the_text_around_it():
    # tokenizer.rs:88-96
    tokenizer = host.Tokenizer(archive(["<|x|>", "a", "b", "ab"], [3, 1, 1, 1], ["a b"]), "whole")
    assert tokenizer.encode("<|x|>ab") == [0, 3]
    assert tokenizer.encode("a<|x|>b") == [1, 0, 2]
    assert tokenizer.piece(3) == b"ab" and tokenizer.piece(0) == b"<|x|>"


def test_the_lowest_ranked_pair_merges_first():
    # tokenizer.rs:98-111
    tokenizer = host.Tokenizer(archive(["a", "b", "c", "bc", "abc"], [1] * 5, ["b c", "a bc"]), "whole")
    assert tokenizer.encode("abc") == [4]
    assert tokenizer.encode("aabc") == [0, 4]
    assert tokenizer.vocabulary() == 5
    assert tokenizer.id("abc") == 4 and tokenizer.id("d") is None


def test_the_rule_of_the_caller_decides_where_the_text_splits():
    # tokenizer.rs:113-121
    source = archive(["hello", "world"], [1, 1], [])
    tokenizer = host.Tokenizer(source, "per_space")
    assert tokenizer.encode("hello world") == [0, 1]
    refuses(lambda: tokenizer.encode("hello  world"), "one of them holds no character")
    refuses(lambda: host.Tokenizer(source, "whole").encode("hello world"), "this vocabulary holds no piece")


def test_what_no_token_spells_and_what_is_no_byte_level_bpe_is_refused():
    # tokenizer.rs:123-154
    tokenizer = host.Tokenizer(archive(["a"], [1], []), "per_character")
    refuses(lambda: tokenizer.encode("b"), "this vocabulary holds no piece b")
    refuses(lambda: tokenizer.piece(1), "this vocabulary holds no token 1 of 1 tokens")
    refuses(lambda: host.Tokenizer(archive(["a"], [1], [], model="bert")), "this gguf names bert as its tokenizer.ggml.model")
    refuses(lambda: host.Tokenizer(archive(["a", "b", "ab"], [1, 1, 1], ["ab"])), "the merge ab of this gguf names two pieces")


def test_text_waits_for_the_bytes_a_character_stands_on():
    # tokenizer.rs:156-165
    text = host.Text()
    assert text.push("We".encode()) == "We"
    assert text.push(bytes([0xE4, 0xB8])) == ""
    assert text.push(bytes([0x96, 0x21])) == "世!"
    assert text.push(bytes([0xFF])) == "�"
    assert text.push(bytes([0xF0, 0x9F])) == ""
    assert text.flush() == "�"
    # what Python's own lossy decoder makes of ill-formed bytes, fed whole and byte by byte
    rng = random.Random(3)
    for _ in range(200):
        raw = bytes(rng.choice([0x41, 0xC3, 0xA9, 0xE4, 0xB8, 0x96, 0xF0, 0x9F, 0x98, 0x80, 0xFF, 0xED, 0xA0, 0x80, 0xC0, 0xF4, 0x90]) for _ in range(12))
        want = raw.decode("utf-8", errors="replace")
        assert text.push(raw) + text.flush() == want
        assert "".join(text.push(bytes([b])) for b in raw) + text.flush() == want
    text.close()


def test_the_qwen_rule_is_the_published_pattern():
    regex = pytest.importorskip("regex")
    pattern = regex.compile(QWEN2_PATTERN)
    samples = ["Hello, world! It's 2024: we'll see what they've done, I'm sure you'd agree, they're here.",
               "  leading spaces and\ttabs\n\n\nthree lines  \n  indented", "price: $12.50 (approx.) -- 3rd time", "DON'T SHOUT, HE'S HERE, WE'LL GO",
               "café naïve 世界你好 مرحبا привет ٣٤", "x = y**2 + foo_bar(baz) # comment\r\n\treturn x;\r\n",
               "emoji \U0001F600\U0001F601 and em spaces  line sep", "a'b 'c ''s 'S 't'T", "trailing   ", "   ", "\n", "", "1234567 89", "!!!\n\n??? \n ...", " \n a",
               "<|im_start|>user\nhi<|im_end|>\n"]
    rng = random.Random(7)
    alphabet = list("ab Z9'\n\r\t .,!?-_") + ["é", "世", "٣", " ", " ", "\U0001F600", "'s", "'ll", "  ", "\n\n"]
    for _ in range(600):
        samples.append("".join(rng.choice(alphabet) for _ in range(rng.randint(1, 24))))
    for sample in samples:
        want = pattern.findall(sample)
        assert "".join(want) == sample  # the pattern leaves no character out
        assert host.rule_pieces("qwen", sample) == want, repr(sample)


def test_a_qwen_style_vocabulary_rounds_text_through_ids():
    # bytes as single tokens plus a few merges and ChatML's control tokens: text -> ids -> text
    alphabet = []
    extra = 0
    for byte in range(256):
        printable = 0x21 <= byte <= 0x7E or 0xA1 <= byte <= 0xAC or 0xAE <= byte <= 0xFF
        alphabet.append(chr(byte) if printable else chr(256 + extra))
        extra += 0 if printable else 1
    merges = ["h e", "l l", "he ll", "hell o", "Ġ w", "Ġw o"]
    tokens = alphabet + ["he", "ll", "hell", "hello", "Ġw", "Ġwo", "<|im_start|>", "<|im_end|>", "<|endoftext|>"]
    kinds = [1] * (len(tokens) - 3) + [3, 3, 3]
    tokenizer = host.Tokenizer(archive(tokens, kinds, merges), "qwen")
    assert tokenizer.encode("hello world") == [259, 261, ord("r"), ord("l"), ord("d")]
    prompt = "<|im_start|>user\nhello wörld 世界! 123<|im_end|>\n<|im_start|>assistant\n"
    ids = tokenizer.encode(prompt)
    assert ids[0] == 262 and ids.count(262) == 2 and ids.count(263) == 1
    assert tokenizer.decode(ids) == prompt
    assert all(id < len(tokens) for id in ids)
