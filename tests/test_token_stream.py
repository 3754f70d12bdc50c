"""Host-side streaming detokeniser against hand-worked cases of the reference's rule
(rai-models/src/llm/mod.rs:50-67): text is released only when the decoded tail grew and ends alphanumerically."""
import pytest

from rai_amd.token_stream import TokenOutputStream, _is_alphanumeric

tokenizers = pytest.importorskip("tokenizers")


@pytest.fixture(scope="module")
def byte_bpe():
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers, trainers

    tok = Tokenizer(models.BPE())
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tok.decoder = decoders.ByteLevel()
    trainer = trainers.BpeTrainer(vocab_size=300, special_tokens=["<|endoftext|>"],
                                  initial_alphabet=pre_tokenizers.ByteLevel.alphabet())
    tok.train_from_iterator(["hello world, hello there", "the quick brown fox"], trainer)
    return tok


def test_multibyte_character_is_held_until_complete(byte_bpe):
    ids = byte_bpe.encode("你", add_special_tokens=False).ids
    assert len(ids) == 3          # one token per UTF-8 byte: nothing in the training text merges them
    s = TokenOutputStream(byte_bpe)
    assert s.is_empty() and len(s) == 0
    assert s.next_token(ids[0]) is None
    assert s.next_token(ids[1]) is None
    assert s.next_token(ids[2]) == "你"
    assert list(s.tokens()) == ids and s.prev_index == 0 and s.current_index == 3


def test_punctuation_waits_for_the_next_word(byte_bpe):
    s = TokenOutputStream(byte_bpe)
    s.prompt("the quick")
    n_prompt = len(s)
    assert (s.prev_index, s.current_index) == (0, n_prompt)
    out = []
    for t in byte_bpe.encode(" fox, hello!", add_special_tokens=False).ids:
        out.append(s.next_token(t))
    pieces = [p for p in out if p is not None]
    # ", " and the final "!" end in non-alphanumerics: the comma and blank come out glued to "hello", "!" never does
    assert "".join(pieces) == " fox, hello"
    assert all(p[-1].isalnum() for p in pieces)
    assert out[-1] is None
    # the cursors moved one emission behind the end: the tail decoded next time starts at the previous emission
    assert s.current_index <= len(s) - 1 and s.prev_index < s.current_index


def test_emitted_text_is_a_prefix_of_the_full_decode(byte_bpe):
    text = " the quick brown fox said héllo wörld 42 times"
    ids = byte_bpe.encode(text, add_special_tokens=False).ids
    s = TokenOutputStream(byte_bpe)
    s.prompt("hello there")
    got = "".join(p for p in (s.next_token(t) for t in ids) if p)
    assert got == text            # ends in a letter, so everything has been released


def test_special_tokens_are_skipped(byte_bpe):
    s = TokenOutputStream(byte_bpe)
    eos = byte_bpe.token_to_id("<|endoftext|>")
    a = byte_bpe.encode("fox", add_special_tokens=False).ids
    assert s.next_token(eos) is None
    assert "".join(p for p in (s.next_token(t) for t in a) if p) == "fox"


def test_alphanumeric_rule():
    for ch in "aZé你5٣ⅷ½":
        assert _is_alphanumeric(ch), ch
    for ch in " ,!\n�-_€":
        assert not _is_alphanumeric(ch), ch
