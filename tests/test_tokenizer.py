"""Byte-pair-encoding tokenizer (reference: plugins/tokenizer-bpe/src/lib.rs, cited TB:line).

Host code: everything but the last test runs without a GPU.

Pins of the oracle (oracle/bpe_oracle.py) and of the library, none of them a retyped formula:
  * the reference's own three tests (TB:393-451), run against both;
  * merge sequences, vocabulary ids and tokenisations worked out by hand on tiny corpora;
  * a brute-force check, with independent counting code, that every learned rule was a most
    frequent pair when it was chosen (any such pair is a valid output of the reference, whose own
    pick follows a randomly seeded hash map, TB:198-201);
  * the decode quirks read off TB:323-337, case by case;
  * Rust's White_Space set against Python's str.split on the characters where the two differ.
The library is then compared with the oracle, exactly, on seeded random corpora and texts
(merge rules, ids, token strings, decoded text), including a tokenizer trained twice, where the
same pair is a rule at two ranks.
"""
import collections
import random

import numpy as np
import pytest

from coeus_amd import BpeTokenizer, BpeTokenizerPlugin, ProcessingError, StringToken
from oracle.bpe_oracle import BpeOracle, split_whitespace

CORPUS = ["the cat sat on the mat", "the dog sat on the log", "the cat and the dog"]  # TB:409-413


def both():
    return BpeTokenizer(), BpeOracle()


def lib_tokens(tok, text):
    return [(t.as_str(), t.id()) for t in tok.tokenize_str(text)]


# ---------------------------------------------------------------- the reference's own tests
@pytest.mark.parametrize("make", [BpeTokenizer, None])
def test_reference_basic(make):  # TB:393-404
    if make:
        tok = make()
        tokens = tok.tokenize_str("hello")
        assert len(tokens) == 5
        assert tok.decode(tokens) == "hello"
    else:
        o = BpeOracle()
        tokens = o.tokenize("hello")
        assert len(tokens) == 5
        assert o.decode([t for t, _ in tokens]) == "hello"


def test_reference_training():  # TB:406-428
    tok, o = both()
    tok.train(CORPUS, 10)
    o.train(CORPUS, 10)
    assert tok.vocab_size() > 256 and o.vocab_size() > 256
    tokens = tok.tokenize_str("the cat")
    assert tokens
    decoded = tok.decode(tokens)
    assert "the" in decoded and "cat" in decoded
    od = o.decode([t for t, _ in o.tokenize("the cat")])
    assert "the" in od and "cat" in od


def test_reference_special_tokens():  # TB:430-451
    tok, o = both()
    for name, i in (("<PAD>", 0), ("<UNK>", 1), ("<BOS>", 2), ("<EOS>", 3)):
        assert tok.contains_token(name) and o.contains_token(name)
        assert tok.id_from_token(name) == i == o.id_from_token(name)


def test_plugin_identity():  # TB:16-51
    p = BpeTokenizerPlugin()
    assert p.id() == "bpe_tokenizer" and p.version() == (0, 1, 0)
    assert set(p.capabilities()) == {"tokenization", "bpe"}
    t = p.create_tokenizer()
    assert isinstance(t, BpeTokenizer) and t.name() == "bpe_tokenizer"


# ---------------------------------------------------------------- the initial vocabulary (TB:117-143)
def test_initial_vocabulary():
    tok, o = both()
    assert tok.vocab_size() == 260 == o.vocab_size()  # 256 byte tokens + 4 special strings
    for b in range(256):
        s = chr(b) if b < 0x80 else "<0x%02X>" % b
        assert tok.id_from_token(s) == b == o.id_from_token(s)
    # the special tokens overwrote ids 0..3 of the id -> string map only
    for i, name in enumerate(["<PAD>", "<UNK>", "<BOS>", "<EOS>"]):
        assert tok.token_from_id(i) == name == o.token_from_id(i)
    assert tok.token_from_id(65) == "A" and tok.token_from_id(0xE9) == "<0xE9>"
    assert tok.token_from_id(256) is None and tok.id_from_token("ab") is None
    assert tok.add_token("zz") == 256 == o.add_token("zz")  # next_id was not moved by the special tokens


# ---------------------------------------------------------------- hand-worked training
def test_training_by_hand():
    # words ab x3, abc x1: (a,b) has 4, (b,c) 1 -> rule 0 = (a,b); then only (ab,c) -> rule 1; then
    # no pair is left and training stops although 10 merges were asked for (TB:236-238)
    for t in both():
        t.train(["ab ab ab", "abc"], 10)
        merges = t.merges() if isinstance(t, BpeTokenizer) else t.merges
        assert [tuple(m) for m in merges] == [("a", "b"), ("ab", "c")]
        assert t.vocab_size() == 262
        assert t.id_from_token("ab") == 256 and t.id_from_token("abc") == 257
    tok, o = both()
    tok.train(["ab ab ab", "abc"], 10)
    o.train(["ab ab ab", "abc"], 10)
    want = [("abc", 257), (" ", 32), ("ab", 256), (" ", 32), ("x", 120), (" ", 32), ("b", 98), ("a", 97)]
    assert lib_tokens(tok, "  abc ab\tx\n ba ") == want == o.tokenize("  abc ab\tx\n ba ")


def test_training_tie_break_and_overlaps():
    # "ab cd": both pairs occur once -> the smaller pair first
    for t in both():
        t.train(["ab cd"], 2)
        merges = t.merges() if isinstance(t, BpeTokenizer) else t.merges
        assert [tuple(m) for m in merges] == [("a", "b"), ("c", "d")]
    # "aaaa": (a,a) is counted at 3 positions (TB:188-191) and merged greedily from the left into
    # [aa, aa]; the second rule is (aa, aa)
    for t in both():
        t.train(["aaaa b"], 5)
        merges = t.merges() if isinstance(t, BpeTokenizer) else t.merges
        assert [tuple(m) for m in merges] == [("a", "a"), ("aa", "aa")]
    tok = BpeTokenizer()
    tok.train(["aaaa b"], 5)
    assert [s for s, _ in lib_tokens(tok, "aaaaa aaa")] == ["aaaa", "a", " ", "aa", "a"]


def count_pairs(words):
    """Independent pair count: words is a Counter of tuples of token strings."""
    c = collections.Counter()
    for w, f in words.items():
        for x, y in zip(w, w[1:]):
            c[(x, y)] += f
    return c


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_every_rule_was_a_most_frequent_pair(seed):
    rng = random.Random(seed)
    corpus = [" ".join("".join(rng.choice("abcé") for _ in range(rng.randint(1, 6))) for _ in range(30))
              for _ in range(4)]
    tok, o = both()
    tok.train(corpus, 25)
    o.train(corpus, 25)
    assert tok.merges() == [tuple(m) for m in o.merges]
    words = collections.Counter()
    for text in corpus:
        for w in text.split():
            words[tuple(chr(b) if b < 0x80 else "<0x%02X>" % b for b in w.encode())] += 1
    for first, second in tok.merges():
        freqs = count_pairs(words)
        assert freqs[(first, second)] == max(freqs.values())
        nxt = collections.Counter()
        for w, f in words.items():
            out, i = [], 0
            while i < len(w):
                if i + 1 < len(w) and (w[i], w[i + 1]) == (first, second):
                    out.append(first + second)
                    i += 2
                else:
                    out.append(w[i])
                    i += 1
            nxt[tuple(out)] += f
        words = nxt


# ---------------------------------------------------------------- white space, UTF-8
def test_white_space_is_rusts():
    seps = ["\u00a0", "\u3000", "\u2003", "\u0085", "\u1680", "\u2028", "\u2029", "\u202f", "\u205f",
            "\u000b", "\u000c", "\u200a", "\r\n"]
    letters = "abcdefghijklmn"
    text = "".join(l + s for l, s in zip(letters, seps + [""]))
    assert split_whitespace(text) == list(letters)
    tok = BpeTokenizer()
    assert [s for s, _ in lib_tokens(tok, text) if s != " "] == list(letters)
    # U+001C..U+001F split in Python's str.split but are not White_Space; neither are U+200B
    # (zero width space), U+180E and U+FEFF
    assert len("a\x1cb".split()) == 2
    for t in ("a\x1cb", "a\x1fb", "a\u200bb", "a\u180eb", "a\ufeffb"):
        assert split_whitespace(t) == [t]
        assert " " not in [s for s, _ in lib_tokens(tok, t)]
    assert lib_tokens(tok, "") == [] and lib_tokens(tok, " \t\n ") == []


def test_non_ascii_bytes_and_invalid_utf8():
    tok, o = both()
    want = [("<0xC3>", 0xC3), ("<0xA9>", 0xA9), ("t", 116), ("<0xC3>", 0xC3), ("<0xA9>", 0xA9)]
    assert lib_tokens(tok, "été") == want == o.tokenize("été")
    assert list(tok.encode("été")) == [0xC3, 0xA9, 116, 0xC3, 0xA9]
    assert tok.encode("été").dtype == np.uint64
    for bad in (b"\xff", b"a\xc3", b"\xc0\x80", b"\xed\xa0\x80", b"\xf4\x90\x80\x80", b"ok \x80"):
        with pytest.raises(ProcessingError, match="not valid UTF-8"):
            tok.tokenize(bad)
        with pytest.raises(ProcessingError, match="not valid UTF-8"):
            tok.train([bad], 1)
    assert lib_tokens(tok, "\U0010ffff")[0] == ("<0xF4>", 0xF4)  # the largest scalar value is fine


# ---------------------------------------------------------------- decode (TB:319-343)
def test_decode_quirks():
    tok = BpeTokenizer()
    cases = [
        (["h", "i"], "hi"),
        (["<0xC3>", "<0xA9>"], "\ufffd\ufffd"),  # each lone byte goes through from_utf8_lossy
        (["<0xC3><0xA9>"], "\ufffd"),         # a merged token: only characters 3..5 are read
        (["<0x41>"], "A"),
        (["<0x41>junk>"], "A"),
        (["<0xZZ>"], "<0xZZ>"),                   # parse failure: copied
        (["<0x1>"], "<0x1>"),                     # "1>" is not a number
        (["<0x+5>"], "\x05"),                     # from_str_radix accepts a sign
        (["<0x-5>"], "<0x-5>"),
        (["<0x>"], "<0x>"),                       # the reference panics here (TB:329)
        (["<0x4"], "<0x4"),
        ([], ""),
        (["", "a", ""], "a"),
    ]
    for toks, want in cases:
        assert tok.decode(toks) == want, toks
        assert BpeOracle.decode(toks) == want, toks
    assert tok.decode([StringToken.with_id("<0x7A>", 5), StringToken("!")]) == "z!"
    # ids 0..3 name the special tokens in the id -> string map, whatever byte produced them
    assert tok.decode_ids(tok.encode("a\x01b")) == "a<UNK>b"
    assert tok.decode(tok.tokenize("a\x01b")) == "a\x01b"
    with pytest.raises(ProcessingError, match="not found"):
        tok.decode_ids([100000])


# ---------------------------------------------------------------- vocabulary (TB:355-386)
def test_vocabulary_operations():
    tok, o = both()
    for t in (tok, o):
        assert t.add_token("a") == 97            # existing: its id
        assert t.add_token("hello") == 256 and t.add_token("hello") == 256
        assert t.add_token("") == 257
        assert t.contains_token("hello") and t.token_from_id(256) == "hello"
        t.remove_token("x")
        assert not t.contains_token("x") and t.token_from_id(120) is None
        assert t.vocab_size() == 261
        assert t.add_token("x") == 258           # a removed token comes back under a new id
        t.remove_token("\x00")                   # shares id 0 with <PAD>: the reverse entry goes too
        assert t.token_from_id(0) is None and t.id_from_token("<PAD>") == 0
    with pytest.raises(ProcessingError, match="Token not found: nope"):
        tok.remove_token("nope")
    with pytest.raises(KeyError):
        o.remove_token("nope")
    tok2, o2 = both()
    tok2.remove_token("b")
    o2.remove_token("b")
    assert lib_tokens(tok2, "abc") == [("a", 97), ("b", 1), ("c", 99)] == o2.tokenize("abc")  # <UNK>


# ---------------------------------------------------------------- library == oracle on random input
ALPHABETS = ["ab", "abcdefgh ", "aé漢  ", "<0x41>PAD "]


@pytest.mark.parametrize("seed", range(6))
def test_library_matches_oracle(seed):
    rng = random.Random(100 + seed)
    alpha = ALPHABETS[seed % len(ALPHABETS)] + " \t"
    def text(n):
        return "".join(rng.choice(alpha) for _ in range(n))
    tok, o = both()
    rounds = 2 if seed % 2 else 1  # trained twice: the same pair becomes a rule at two ranks
    for r in range(rounds):
        corpus = [text(rng.randint(0, 200)) for _ in range(rng.randint(1, 5))]
        nm = rng.randint(0, 40)
        tok.train(corpus, nm)
        o.train(corpus, nm)
        assert tok.merges() == [tuple(m) for m in o.merges]
        assert tok.vocab_size() == o.vocab_size()
    for _ in range(30):
        t = text(rng.randint(0, 120))
        got = lib_tokens(tok, t)
        want = o.tokenize(t)
        assert got == want, t
        assert list(tok.encode(t)) == [i for _, i in want]
        assert tok.decode([s for s, _ in got]) == BpeOracle.decode([s for s, _ in want])
    for i in range(o.next_id + 2):
        assert tok.token_from_id(i) == o.token_from_id(i)


def test_same_pair_at_two_ranks():
    # training again starts from bytes (TB:169-181), so the same corpus teaches the same rules a
    # second time; bpe() walks all of them in order (TB:250), and the later copy of a rule can
    # fire on tokens that a rule between the two copies produced
    tok, o = both()
    for t in (tok, o):
        t.train(["ab ab ab abc abc xab"], 2)   # (a,b), (ab,c)
        t.train(["xa xa xa xa ab"], 1)         # (x,a): now "xab" -> [xa, b]
        t.train(["ab ab ab abc abc"], 2)       # (a,b), (ab,c) again
    assert tok.merges() == [("a", "b"), ("ab", "c"), ("x", "a"), ("a", "b"), ("ab", "c")] == [tuple(m) for m in o.merges]
    for text in ("xab", "abc xabc ab", "xaab"):
        assert lib_tokens(tok, text) == o.tokenize(text)
    assert [s for s, _ in lib_tokens(tok, "xab")] == ["x", "ab"]      # rule 0 fires before rule 2 can
    assert [s for s, _ in lib_tokens(tok, "xaab")] == ["xa", "ab"]    # rule 2, then the second (a,b)


def test_tokenize_decode_round_trip_property():
    # ASCII words separated by single spaces survive tokenize -> decode whatever was learned
    tok = BpeTokenizer()
    tok.train(CORPUS * 3, 60)
    for t in ("the cat sat", "a", "dog log mat the the", "unseen words zebra"):
        assert tok.decode(tok.tokenize(t)) == t
    assert tok.decode(tok.tokenize("  the \n cat ")) == "the cat"
    # a whole word learned as one token
    assert any(s == "the" for s, _ in lib_tokens(tok, "the"))
    assert len(tok.tokenize("the")) == 1


# ---------------------------------------------------------------- text -> ids -> logits -> text
@pytest.mark.gpu
def test_text_to_model_to_text():
    from coeus_amd import BasicGenerationConfig, Transformer250MConfig, TransformerModelBuilder

    tok = BpeTokenizer()
    tok.train(CORPUS, 20)
    cfg = Transformer250MConfig(hidden_dim=64, num_layers=2, num_heads=4, intermediate_dim=128,
                                vocab_size=tok.vocab_size(), max_seq_len=64, norm_scope="token")
    model = TransformerModelBuilder().build(cfg, seed=7)
    ids = tok.encode("the cat sat on")
    logits = model.forward(ids)
    assert logits.shape == (tok.vocab_size(),) and np.isfinite(logits).all()
    assert np.array_equal(logits, model.forward([int(i) for i in ids]))
    new = model.generate(ids, BasicGenerationConfig(max_length=8, temperature=0.0))
    assert len(new) == 8 and all(0 <= i < tok.vocab_size() for i in new)
    assert new[0] == int(np.argmax(logits))
    known = [i for i in new if tok.token_from_id(i) is not None]
    assert isinstance(tok.decode_ids(known), str)
