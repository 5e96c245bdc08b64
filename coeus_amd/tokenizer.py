"""Host-side mirror of the reference's byte-pair-encoding tokenizer plugin:

    BpeTokenizerPlugin().create_tokenizer() -> tokenizer;  tokenizer.tokenize_str(text) -> tokens

(rustllm-core/plugins/tokenizer-bpe/src/lib.rs:16-51, 100-386, over the traits of
rustllm-core/src/core/tokenizer.rs:17-72, 119-160), implemented over the C ABI of
libcoeus_mi355x.so (coeus_bpe_*).  Names, argument meaning and error behaviour follow the
reference; `Result<T>` becomes "return T or raise", `Option<T>` becomes "T or None".
"""
import ctypes as C

import numpy as np

from . import _lib
from .plugin import ProcessingError, _check


class StringToken:
    """StringToken (core/tokenizer.rs:29-72): a token string with an optional id."""

    __slots__ = ("value", "_id")

    def __init__(self, value, id=None):
        self.value = value
        self._id = id

    @classmethod
    def with_id(cls, value, id):
        return cls(value, id)

    def id(self):
        return 0 if self._id is None else self._id  # core/tokenizer.rs:61-63

    def as_str(self):
        return self.value

    def as_bytes(self):
        return self.value.encode("utf-8")

    def __len__(self):
        return len(self.as_bytes())

    def __eq__(self, other):
        return isinstance(other, StringToken) and (self.value, self._id) == (other.value, other._id)

    def __repr__(self):
        return f"StringToken({self.value!r}, id={self._id})"


def _text(s):
    """A str as UTF-8 bytes; bytes are passed through (the library rejects invalid UTF-8)."""
    return s if isinstance(s, (bytes, bytearray)) else s.encode("utf-8", "surrogatepass")


class BpeTokenizerPlugin:
    """BpeTokenizerPlugin (tokenizer-bpe/src/lib.rs:16-51)."""

    def id(self):
        return "bpe_tokenizer"

    def version(self):
        return (0, 1, 0)

    def capabilities(self):
        return ("tokenization", "bpe")

    def create_tokenizer(self):
        return BpeTokenizer()


class BpeTokenizer:
    """BpeTokenizer (tokenizer-bpe/src/lib.rs:100-386)."""

    def __init__(self):
        self._h = C.c_void_p()
        _check(_lib.load().coeus_bpe_create(C.byref(self._h)))

    # ---- BpeTokenizer
    def train(self, corpus, num_merges):
        """train(&mut self, corpus, num_merges) (lib.rs:167-240)."""
        raw = [bytes(_text(t)) for t in corpus]
        arr = (C.c_char_p * max(1, len(raw)))(*raw)
        lens = (C.c_uint64 * max(1, len(raw)))(*[len(r) for r in raw])
        _check(_lib.load().coeus_bpe_train(self._h, arr, lens, len(raw), int(num_merges)))

    def merges(self):
        """The merge rules learned so far, as (first, second) strings (lib.rs:107)."""
        lib = _lib.load()
        out = []
        for i in range(lib.coeus_bpe_num_merges(self._h)):
            l1, l2 = C.c_uint64(), C.c_uint64()
            _check(lib.coeus_bpe_merge_rule(self._h, i, None, 0, C.byref(l1), None, 0, C.byref(l2)))
            b1, b2 = C.create_string_buffer(max(1, l1.value)), C.create_string_buffer(max(1, l2.value))
            _check(lib.coeus_bpe_merge_rule(self._h, i, b1, l1.value, C.byref(l1), b2, l2.value, C.byref(l2)))
            out.append((b1.raw[:l1.value].decode("utf-8"), b2.raw[:l2.value].decode("utf-8")))
        return out

    # ---- Tokenizer
    def _tokenize(self, text, want_pieces):
        lib = _lib.load()
        raw = bytes(_text(text))
        n, nb = C.c_uint64(), C.c_uint64()
        _check(lib.coeus_bpe_tokenize(self._h, raw, len(raw), None, 0, C.byref(n), None, 0, None, C.byref(nb)))
        ids = np.zeros(n.value, dtype=np.uint64)
        if not want_pieces:
            _check(lib.coeus_bpe_tokenize(self._h, raw, len(raw), ids.ctypes.data, n.value, C.byref(n),
                                          None, 0, None, C.byref(nb)))
            return ids, None, None
        pieces = C.create_string_buffer(max(1, nb.value))
        offs = np.zeros(n.value + 1, dtype=np.uint64)
        _check(lib.coeus_bpe_tokenize(self._h, raw, len(raw), ids.ctypes.data, n.value, C.byref(n),
                                      pieces, nb.value, offs.ctypes.data, C.byref(nb)))
        return ids, pieces.raw[:nb.value], offs

    def tokenize(self, text):
        """tokenize(input) (lib.rs:285-317): the list of StringToken (the reference returns an iterator)."""
        ids, pieces, offs = self._tokenize(text, True)
        return [StringToken.with_id(pieces[int(offs[i]):int(offs[i + 1])].decode("utf-8"), int(ids[i]))
                for i in range(len(ids))]

    tokenize_str = tokenize  # core/tokenizer.rs:132-134

    def encode(self, text):
        """The ids of tokenize(text) as a uint64 array, ready for TransformerModel.forward."""
        return self._tokenize(text, False)[0]

    def decode(self, tokens):
        """decode(tokens) (lib.rs:319-343): works on the token strings, as the reference does."""
        raw = [t.as_bytes() if isinstance(t, StringToken) else bytes(_text(t)) for t in tokens]
        offs = np.zeros(len(raw) + 1, dtype=np.uint64)
        np.cumsum([len(r) for r in raw], out=offs[1:]) if raw else None
        blob = b"".join(raw)
        n = C.c_uint64()
        lib = _lib.load()
        _check(lib.coeus_bpe_decode(blob, offs.ctypes.data, len(raw), None, 0, C.byref(n)))
        out = C.create_string_buffer(max(1, n.value))
        _check(lib.coeus_bpe_decode(blob, offs.ctypes.data, len(raw), out, n.value, C.byref(n)))
        return out.raw[:n.value].decode("utf-8")

    def decode_ids(self, ids):
        """token_from_id for every id, then decode.  An id without an entry raises; ids 0..3 name
        the special tokens, which took those slots of the id -> string map (lib.rs:159-164)."""
        toks = []
        for i in ids:
            t = self.token_from_id(int(i))
            if t is None:
                raise ProcessingError(f"Token id not found: {int(i)}")
            toks.append(t)
        return self.decode(toks)

    def vocab_size(self):
        return int(_lib.load().coeus_bpe_vocab_size(self._h))

    def name(self):
        return "bpe_tokenizer"

    # ---- VocabularyTokenizer (lib.rs:355-386)
    def add_token(self, token):
        raw, i = bytes(_text(token)), C.c_uint64()
        _check(_lib.load().coeus_bpe_add_token(self._h, raw, len(raw), C.byref(i)))
        return int(i.value)

    def remove_token(self, token):
        raw = bytes(_text(token))
        _check(_lib.load().coeus_bpe_remove_token(self._h, raw, len(raw)))

    def contains_token(self, token):
        return self.id_from_token(token) is not None

    def id_from_token(self, token):
        raw, i, found = bytes(_text(token)), C.c_uint64(), C.c_int()
        _check(_lib.load().coeus_bpe_id_from_token(self._h, raw, len(raw), C.byref(i), C.byref(found)))
        return int(i.value) if found.value else None

    def token_from_id(self, id):
        lib = _lib.load()
        n, found = C.c_uint64(), C.c_int()
        _check(lib.coeus_bpe_token_from_id(self._h, int(id), None, 0, C.byref(n), C.byref(found)))
        if not found.value:
            return None
        out = C.create_string_buffer(max(1, n.value))
        _check(lib.coeus_bpe_token_from_id(self._h, int(id), out, n.value, C.byref(n), C.byref(found)))
        return out.raw[:n.value].decode("utf-8")

    def close(self):
        if self._h:
            _lib.load().coeus_bpe_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
