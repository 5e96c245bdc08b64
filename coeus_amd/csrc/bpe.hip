// Byte-pair-encoding tokenizer: the step that turns text into the ids the model consumes.
// Host code only (string work; nothing here touches the device).
//
// Behaviour follows rustllm-core/plugins/tokenizer-bpe/src/lib.rs (TB:line) exactly, quirks
// included, on a different representation: token strings are interned once and words are
// vectors of small integers; a merge rule is (first, second, merged) in those integers, and a
// hash map from a pair to the ranks at which it is a rule replaces the reference's scan over
// every rule for every word.
//
//   Bpe::Bpe           TB:117-143  256 byte tokens, bytes >= 0x80 spelled "<0xNN>"; the four special
//                                  tokens then take ids 0..3 in the id -> string map as well
//   train              TB:167-240  (ties between equally frequent pairs: smallest pair in byte
//                                  order; the reference's choice follows a randomly seeded hash map)
//   apply_merges       TB:243-271  rules in the order learned, each one left-to-right pass.  A pass
//                                  is skipped when its pair is absent, which is decided by looking
//                                  up the ranks of the pairs that ARE present: the lowest rank
//                                  above the last one applied is the next pass that changes anything
//   tokenize           TB:285-317
//   decode_pieces      TB:319-343
#include <algorithm>
#include <array>
#include <cstring>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.hpp"

namespace coeus {

// Decodes one UTF-8 scalar value the way Rust's str validation accepts it (no overlong forms,
// no surrogates, at most U+10FFFF).  Returns its length in bytes, 0 if the bytes are not valid.
static int utf8_next(const unsigned char *p, const unsigned char *end, uint32_t *cp) {
    const unsigned c = p[0];
    if (c < 0x80) { *cp = c; return 1; }
    int n;
    uint32_t v, lo;
    if (c >= 0xC2 && c <= 0xDF) { n = 2; v = c & 0x1F; lo = 0x80; }
    else if (c >= 0xE0 && c <= 0xEF) { n = 3; v = c & 0x0F; lo = 0x800; }
    else if (c >= 0xF0 && c <= 0xF4) { n = 4; v = c & 0x07; lo = 0x10000; }
    else return 0;
    if (end - p < n) return 0;
    for (int i = 1; i < n; i++) {
        if ((p[i] & 0xC0) != 0x80) return 0;
        v = (v << 6) | (p[i] & 0x3F);
    }
    if (v < lo || v > 0x10FFFF || (v >= 0xD800 && v <= 0xDFFF)) return 0;
    *cp = v;
    return n;
}

// char::is_whitespace: the Unicode White_Space property (str::split_whitespace, TB:291).
static bool is_white_space(uint32_t c) {
    return (c >= 0x09 && c <= 0x0D) || c == 0x20 || c == 0x85 || c == 0xA0 || c == 0x1680 ||
           (c >= 0x2000 && c <= 0x200A) || c == 0x2028 || c == 0x2029 || c == 0x202F ||
           c == 0x205F || c == 0x3000;
}

// Calls f(begin, end) for every maximal run of non-white-space characters; false if the text
// is not valid UTF-8 (a Rust &str cannot hold such text, so the reference never sees it).
template <typename F>
static bool for_each_word(const char *text, uint64_t len, F f) {
    const unsigned char *p = (const unsigned char *)text, *end = p + len, *word = nullptr;
    while (p < end) {
        uint32_t cp;
        const int n = utf8_next(p, end, &cp);
        if (n == 0) return false;
        if (is_white_space(cp)) {
            if (word) f(word, p);
            word = nullptr;
        } else if (!word) {
            word = p;
        }
        p += n;
    }
    if (word) f(word, end);
    return true;
}

struct Bpe {
    std::vector<std::string> strs;                      // interned token strings
    std::unordered_map<std::string, uint32_t> intern;   // string -> index into strs
    std::unordered_map<std::string, uint32_t> vocab;    // TB:103 string -> id
    std::unordered_map<uint32_t, std::string> reverse;  // TB:105 id -> string
    std::vector<std::array<uint32_t, 3>> merges;        // TB:107 (first, second, merged), interned
    std::unordered_map<uint64_t, std::vector<uint32_t>> ranks;  // pair -> ascending rule indices
    std::vector<int64_t> public_id;                     // interned index -> vocab id, -1 if absent
    uint32_t next_id = 0;                               // TB:111
    uint32_t byte_tok[256];

    uint32_t intern_str(const std::string &s) {
        auto it = intern.find(s);
        if (it != intern.end()) return it->second;
        const uint32_t i = (uint32_t)strs.size();
        strs.push_back(s);
        intern.emplace(s, i);
        public_id.push_back(-1);
        return i;
    }
    void refresh(uint32_t i) {
        auto it = vocab.find(strs[i]);
        public_id[i] = it == vocab.end() ? -1 : (int64_t)it->second;
    }
    uint32_t add_to_vocab(const std::string &s) {  // TB:146-156
        const uint32_t si = intern_str(s);
        auto it = vocab.find(s);
        if (it != vocab.end()) return it->second;
        const uint32_t id = next_id++;
        vocab.emplace(s, id);
        reverse[id] = s;
        refresh(si);
        return id;
    }
    void add_special(const std::string &s, uint32_t id) {  // TB:159-164
        const uint32_t si = intern_str(s);
        vocab[s] = id;
        reverse[id] = s;
        refresh(si);
    }
    Bpe() {
        for (int b = 0; b < 256; b++) {
            std::string s;
            if (b < 0x80) s.assign(1, (char)b);
            else { char buf[8]; snprintf(buf, sizeof buf, "<0x%02X>", b); s = buf; }
            add_to_vocab(s);
            byte_tok[b] = intern.at(s);
        }
        add_special("<PAD>", 0);
        add_special("<UNK>", 1);
        add_special("<BOS>", 2);
        add_special("<EOS>", 3);
    }
    static uint64_t pair_key(uint32_t a, uint32_t b) { return ((uint64_t)a << 32) | b; }
    void push_merge(uint32_t a, uint32_t b) {
        const std::string merged = strs[a] + strs[b];
        add_to_vocab(merged);
        const uint32_t m = intern.at(merged);
        ranks[pair_key(a, b)].push_back((uint32_t)merges.size());
        merges.push_back({a, b, m});
    }
    // one left-to-right pass of rule (a, b) -> m (TB:251-263)
    static void merge_pass(std::vector<uint32_t> &t, uint32_t a, uint32_t b, uint32_t m) {
        size_t o = 0;
        for (size_t i = 0; i < t.size();) {
            if (i + 1 < t.size() && t[i] == a && t[i + 1] == b) { t[o++] = m; i += 2; }
            else t[o++] = t[i++];
        }
        t.resize(o);
    }
    void apply_merges(std::vector<uint32_t> &t) const {
        int64_t last = -1;
        while (t.size() >= 2) {
            int64_t best = -1;
            for (size_t i = 0; i + 1 < t.size(); i++) {
                auto it = ranks.find(pair_key(t[i], t[i + 1]));
                if (it == ranks.end()) continue;
                // the first rule index above `last` for this pair
                auto r = std::upper_bound(it->second.begin(), it->second.end(), last,
                                          [](int64_t v, uint32_t e) { return v < (int64_t)e; });
                if (r != it->second.end() && (best < 0 || (int64_t)*r < best)) best = *r;
            }
            if (best < 0) break;
            merge_pass(t, merges[best][0], merges[best][1], merges[best][2]);
            last = best;
        }
    }
    void word_tokens(const unsigned char *b, const unsigned char *e, std::vector<uint32_t> &t) const {
        t.clear();
        for (; b < e; b++) t.push_back(byte_tok[*b]);
    }

    bool train(const char *const *texts, const uint64_t *lens, uint64_t n_texts, uint64_t num_merges) {
        std::map<std::vector<uint32_t>, uint64_t> word_freqs;
        std::vector<uint32_t> t;
        for (uint64_t i = 0; i < n_texts; i++) {
            const bool ok = for_each_word(texts[i], lens[i], [&](const unsigned char *b, const unsigned char *e) {
                word_tokens(b, e, t);
                word_freqs[t] += 1;
            });
            if (!ok) return false;
        }
        for (uint64_t it = 0; it < num_merges; it++) {
            std::unordered_map<uint64_t, uint64_t> pair_freqs;
            for (const auto &wf : word_freqs)
                for (size_t i = 0; i + 1 < wf.first.size(); i++)
                    pair_freqs[pair_key(wf.first[i], wf.first[i + 1])] += wf.second;
            if (pair_freqs.empty()) break;
            uint64_t best_key = 0, best_freq = 0;
            bool have = false;
            for (const auto &pf : pair_freqs) {
                bool better = !have || pf.second > best_freq;
                if (have && pf.second == best_freq) {
                    const std::string &a0 = strs[pf.first >> 32], &b0 = strs[best_key >> 32];
                    const int c = a0.compare(b0);
                    better = c < 0 || (c == 0 && strs[(uint32_t)pf.first].compare(strs[(uint32_t)best_key]) < 0);
                }
                if (better) { best_key = pf.first; best_freq = pf.second; have = true; }
            }
            const uint32_t a = (uint32_t)(best_key >> 32), b = (uint32_t)best_key;
            push_merge(a, b);
            const uint32_t m = merges.back()[2];
            std::map<std::vector<uint32_t>, uint64_t> next;
            for (const auto &wf : word_freqs) {
                t = wf.first;
                merge_pass(t, a, b, m);
                next[t] += wf.second;
            }
            word_freqs.swap(next);
        }
        return true;
    }
};

}  // namespace coeus

using namespace coeus;

struct coeus_bpe { Bpe t; };

// copies `s` to a caller buffer under the sizing protocol of the header
static int copy_out(const std::string &s, char *out, uint64_t cap, uint64_t *len) {
    if (len) *len = s.size();
    if (!out) return COEUS_OK;
    if (cap < s.size()) return fail(COEUS_INVALID_INPUT, "output buffer too small: %llu bytes needed",
                                    (unsigned long long)s.size());
    memcpy(out, s.data(), s.size());
    return COEUS_OK;
}

extern "C" {

int coeus_bpe_create(coeus_bpe **out) {
    COEUS_GUARD_BEGIN
    if (!out) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    *out = new coeus_bpe();
    return COEUS_OK;
    COEUS_GUARD_END
}

void coeus_bpe_destroy(coeus_bpe *t) { delete t; }

int coeus_bpe_train(coeus_bpe *t, const char *const *texts, const uint64_t *lens, uint64_t n_texts,
                    uint64_t num_merges) {
    COEUS_GUARD_BEGIN
    if (!t || (n_texts && (!texts || !lens))) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    for (uint64_t i = 0; i < n_texts; i++)
        if (!texts[i] && lens[i]) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (!t->t.train(texts, lens, n_texts, num_merges))
        return fail(COEUS_INVALID_INPUT, "corpus text is not valid UTF-8");
    return COEUS_OK;
    COEUS_GUARD_END
}

int coeus_bpe_tokenize(const coeus_bpe *t, const char *text, uint64_t len, uint64_t *ids,
                       uint64_t ids_cap, uint64_t *n_tokens, char *pieces, uint64_t pieces_cap,
                       uint64_t *offsets, uint64_t *pieces_len) {
    COEUS_GUARD_BEGIN
    if (!t || (!text && len)) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    const Bpe &b = t->t;
    std::vector<uint32_t> all, w;
    const uint32_t space = b.byte_tok[' '];
    const bool ok = for_each_word(text, len, [&](const unsigned char *s, const unsigned char *e) {
        b.word_tokens(s, e, w);
        b.apply_merges(w);
        if (!all.empty()) all.push_back(0xffffffffu);  // the " " token between words (TB:308)
        all.insert(all.end(), w.begin(), w.end());
    });
    if (!ok) return fail(COEUS_INVALID_INPUT, "input text is not valid UTF-8");
    uint64_t bytes = 0;
    for (uint32_t x : all) bytes += x == 0xffffffffu ? 1 : b.strs[x].size();
    if (n_tokens) *n_tokens = all.size();
    if (pieces_len) *pieces_len = bytes;
    if (ids && ids_cap < all.size())
        return fail(COEUS_INVALID_INPUT, "id buffer too small: %llu tokens", (unsigned long long)all.size());
    if (pieces && pieces_cap < bytes)
        return fail(COEUS_INVALID_INPUT, "output buffer too small: %llu bytes needed", (unsigned long long)bytes);
    uint64_t off = 0;
    for (size_t i = 0; i < all.size(); i++) {
        const bool sp = all[i] == 0xffffffffu;
        const uint32_t x = sp ? space : all[i];
        // the separator carries id 32 whatever the vocabulary says (TB:308); a token whose
        // string has left the vocabulary maps to 1 = <UNK> (TB:303-304)
        if (ids) ids[i] = sp ? 32u : (b.public_id[x] < 0 ? 1u : (uint64_t)b.public_id[x]);
        if (offsets) offsets[i] = off;
        if (pieces) memcpy(pieces + off, b.strs[x].data(), b.strs[x].size());
        off += b.strs[x].size();
    }
    if (offsets) offsets[all.size()] = off;
    return COEUS_OK;
    COEUS_GUARD_END
}

int coeus_bpe_decode(const char *pieces, const uint64_t *offsets, uint64_t n_tokens, char *out,
                     uint64_t cap, uint64_t *len) {
    COEUS_GUARD_BEGIN
    if (n_tokens && (!pieces || !offsets)) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    std::string res;
    auto hex = [](char c) { return c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : c >= 'A' && c <= 'F' ? c - 'A' + 10 : -1; };
    for (uint64_t i = 0; i < n_tokens; i++) {
        if (offsets[i + 1] < offsets[i]) return fail(COEUS_INVALID_INPUT, "token offsets must not decrease");
        const char *s = pieces + offsets[i];
        const uint64_t n = offsets[i + 1] - offsets[i];
        bool done = false;
        if (n >= 5 && s[0] == '<' && s[1] == '0' && s[2] == 'x' && s[n - 1] == '>') {
            // u8::from_str_radix(&s[3..5], 16) (TB:329): two digits, or '+' and one digit
            const int h1 = hex(s[4]);
            const int h0 = s[3] == '+' ? 0 : hex(s[3]);
            if (h0 >= 0 && h1 >= 0) {
                const unsigned byte = (unsigned)(h0 * 16 + h1);
                if (byte < 0x80) res.push_back((char)byte);
                else res += "\xEF\xBF\xBD";  // String::from_utf8_lossy of a lone byte: U+FFFD
                done = true;
            }
        }
        if (!done) res.append(s, n);
    }
    return copy_out(res, out, cap, len);
    COEUS_GUARD_END
}

uint64_t coeus_bpe_vocab_size(const coeus_bpe *t) { return t ? t->t.vocab.size() : 0; }
uint64_t coeus_bpe_num_merges(const coeus_bpe *t) { return t ? t->t.merges.size() : 0; }

int coeus_bpe_merge_rule(const coeus_bpe *t, uint64_t index, char *first, uint64_t first_cap,
                         uint64_t *first_len, char *second, uint64_t second_cap, uint64_t *second_len) {
    COEUS_GUARD_BEGIN
    if (!t) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    if (index >= t->t.merges.size())
        return fail(COEUS_INVALID_INPUT, "merge rule %llu out of range [0, %llu)", (unsigned long long)index,
                    (unsigned long long)t->t.merges.size());
    const auto &m = t->t.merges[index];
    COEUS_TRY(copy_out(t->t.strs[m[0]], first, first_cap, first_len));
    return copy_out(t->t.strs[m[1]], second, second_cap, second_len);
    COEUS_GUARD_END
}

int coeus_bpe_add_token(coeus_bpe *t, const char *token, uint64_t len, uint64_t *id_out) {
    COEUS_GUARD_BEGIN
    if (!t || (!token && len)) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    const uint32_t id = t->t.add_to_vocab(std::string(token ? token : "", len));
    if (id_out) *id_out = id;
    return COEUS_OK;
    COEUS_GUARD_END
}

int coeus_bpe_remove_token(coeus_bpe *t, const char *token, uint64_t len) {
    COEUS_GUARD_BEGIN
    if (!t || (!token && len)) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    const std::string s(token ? token : "", len);
    auto it = t->t.vocab.find(s);
    if (it == t->t.vocab.end()) return fail(COEUS_INVALID_INPUT, "Token not found: %s", s.c_str());  // TB:369-372
    t->t.reverse.erase(it->second);
    t->t.vocab.erase(it);
    auto si = t->t.intern.find(s);
    if (si != t->t.intern.end()) t->t.refresh(si->second);
    return COEUS_OK;
    COEUS_GUARD_END
}

int coeus_bpe_id_from_token(const coeus_bpe *t, const char *token, uint64_t len, uint64_t *id_out,
                            int *found) {
    COEUS_GUARD_BEGIN
    if (!t || (!token && len) || !found) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    auto it = t->t.vocab.find(std::string(token ? token : "", len));
    *found = it != t->t.vocab.end();
    if (*found && id_out) *id_out = it->second;
    return COEUS_OK;
    COEUS_GUARD_END
}

int coeus_bpe_token_from_id(const coeus_bpe *t, uint64_t id, char *out, uint64_t cap, uint64_t *len,
                            int *found) {
    COEUS_GUARD_BEGIN
    if (!t || !found) return fail(COEUS_INVALID_INPUT, "null pointer argument");
    auto it = id <= 0xffffffffull ? t->t.reverse.find((uint32_t)id) : t->t.reverse.end();
    *found = it != t->t.reverse.end();
    if (!*found) { if (len) *len = 0; return COEUS_OK; }
    return copy_out(it->second, out, cap, len);
    COEUS_GUARD_END
}

}  // extern "C"
