"""CPU restatement of the reference's byte-pair-encoding tokenizer (pure Python, dictionaries).

TEST INFRASTRUCTURE ONLY: imported by tests/.  Nothing under coeus_amd/ imports this module.

Follows rustllm-core/plugins/tokenizer-bpe/src/lib.rs (cited as TB:line) statement by statement,
on the same data structures (token strings in hash maps, merges as pairs of strings), so it is
slow and obviously the same algorithm:

  BpeOracle()            TB:117-143  256 byte tokens (bytes >= 0x80 spelled "<0xNN>"), then the four
                                     special tokens inserted OVER ids 0..3 of the reverse map
  add_to_vocab           TB:146-156
  add_special_token      TB:159-164
  train                  TB:167-240
  bpe                    TB:243-271  every merge rule, in the order learned, as one left-to-right pass
  tokenize               TB:285-317  split on Unicode white space, bytes -> tokens -> bpe -> ids
                                     (unknown -> 1), a " " token (id 32) between words
  decode                 TB:319-343  concatenates token strings; a string of the form "<0x..>" is
                                     read as ONE byte taken from its characters 3..5
  vocabulary queries     TB:355-386

Two places where the reference's behaviour is not a function of its inputs or is a panic:
  * train picks `pair_freqs.iter().max_by_key(freq)` (TB:198-201) over a HashMap with a randomly
    seeded hasher: among pairs of equal, maximal frequency ANY may win, differently on every run.
    This restatement (and the library) take the smallest (first, second) in byte order.
  * decode slices `s[3..5]` (TB:329) and panics for a token like "<0x>"; here that token is
    copied as it is, like any other that fails the hexadecimal parse.

Pinned by: the reference's own three tests (TB:393-451) in tests/test_tokenizer.py, hand-worked
merge sequences on tiny corpora, and a brute-force check that every learned pair had maximal
frequency when it was chosen.
"""

# char::is_whitespace = the Unicode White_Space property (what str::split_whitespace uses)
WHITE_SPACE = frozenset(
    list(range(0x09, 0x0E)) + [0x20, 0x85, 0xA0, 0x1680] + list(range(0x2000, 0x200B)) +
    [0x2028, 0x2029, 0x202F, 0x205F, 0x3000])


def split_whitespace(text):
    """str::split_whitespace: maximal runs of non-white-space characters."""
    words, cur = [], []
    for ch in text:
        if ord(ch) in WHITE_SPACE:
            if cur:
                words.append("".join(cur))
                cur = []
        else:
            cur.append(ch)
    if cur:
        words.append("".join(cur))
    return words


def byte_token(b):
    """TB:129-132: String::from_utf8(vec![b]) succeeds for ASCII only."""
    return chr(b) if b < 0x80 else "<0x%02X>" % b


class BpeOracle:
    def __init__(self):
        self.vocab = {}          # token string -> id
        self.reverse_vocab = {}  # id -> token string
        self.merges = []         # (first, second)
        self.special_tokens = {}
        self.next_id = 0
        for b in range(256):
            self.add_to_vocab(byte_token(b))
        self.add_special_token("<PAD>", 0)
        self.add_special_token("<UNK>", 1)
        self.add_special_token("<BOS>", 2)
        self.add_special_token("<EOS>", 3)

    def add_to_vocab(self, token):
        if token in self.vocab:
            return self.vocab[token]
        i = self.next_id
        self.vocab[token] = i
        self.reverse_vocab[i] = token
        self.next_id += 1
        return i

    def add_special_token(self, token, i):
        self.vocab[token] = i
        self.reverse_vocab[i] = token
        self.special_tokens[token] = i
        return i

    def train(self, corpus, num_merges):
        word_freqs = {}
        for text in corpus:
            for word in split_whitespace(text):
                toks = tuple(byte_token(b) for b in word.encode("utf-8"))
                word_freqs[toks] = word_freqs.get(toks, 0) + 1
        for _ in range(num_merges):
            pair_freqs = {}
            for word, freq in word_freqs.items():
                if len(word) < 2:
                    continue
                for i in range(len(word) - 1):
                    p = (word[i], word[i + 1])
                    pair_freqs[p] = pair_freqs.get(p, 0) + freq
            if not pair_freqs:
                break
            best = min(pair_freqs, key=lambda p: (-pair_freqs[p], p[0].encode(), p[1].encode()))
            self.merges.append(best)
            merged = best[0] + best[1]
            self.add_to_vocab(merged)
            new_word_freqs = {}
            for word, freq in word_freqs.items():
                new_word, i = [], 0
                while i < len(word):
                    if i < len(word) - 1 and word[i] == best[0] and word[i + 1] == best[1]:
                        new_word.append(merged)
                        i += 2
                    else:
                        new_word.append(word[i])
                        i += 1
                new_word = tuple(new_word)
                new_word_freqs[new_word] = new_word_freqs.get(new_word, 0) + freq
            word_freqs = new_word_freqs

    def bpe(self, word):
        if len(word) < 2:
            return list(word)
        tokens = list(word)
        for first, second in self.merges:
            new_tokens, i = [], 0
            while i < len(tokens):
                if i < len(tokens) - 1 and tokens[i] == first and tokens[i + 1] == second:
                    new_tokens.append(first + second)
                    i += 2
                else:
                    new_tokens.append(tokens[i])
                    i += 1
            tokens = new_tokens
        return tokens

    def tokenize(self, text):
        """Returns [(token string, id)]."""
        out = []
        for word in split_whitespace(text):
            for t in self.bpe([byte_token(b) for b in word.encode("utf-8")]):
                out.append((t, self.vocab.get(t, 1)))
            out.append((" ", 32))
        if out:
            out.pop()
        return out

    @staticmethod
    def decode(token_strings):
        """Returns the decoded text as a str (a lone byte >= 0x80 becomes U+FFFD, TB:331)."""
        res = []
        for s in token_strings:
            if s.startswith("<0x") and s.endswith(">") and len(s) >= 5:
                try:
                    h = s[3:5]
                    if not all(c in "0123456789abcdefABCDEF" for c in h) and not (
                            h[0] == "+" and h[1] in "0123456789abcdefABCDEF"):
                        raise ValueError(h)
                    byte = int(h, 16)  # u8::from_str_radix accepts a leading '+'
                    res.append(bytes([byte]).decode("utf-8", errors="replace"))
                except ValueError:
                    res.append(s)
            else:
                res.append(s)
        return "".join(res)

    # VocabularyTokenizer (TB:355-386)
    def add_token(self, token):
        return self.add_to_vocab(token)

    def remove_token(self, token):
        if token not in self.vocab:
            raise KeyError("Token not found: %s" % token)
        i = self.vocab.pop(token)
        self.reverse_vocab.pop(i, None)

    def contains_token(self, token):
        return token in self.vocab

    def token_from_id(self, i):
        return self.reverse_vocab.get(i)

    def id_from_token(self, token):
        return self.vocab.get(token)

    def vocab_size(self):
        return len(self.vocab)
