// The byte-pair-encoding tokenizer of J/Tokenizer.java on the host: tokenizer.bin reader, bpe_encode, bpe_decode.
// No GPU code here.  J/ = src/main/java/com/lastbot/llama2j/.
//
// The reference works on Java strings, so every comparison here is on UTF-16 code units: the per-character
// lookup walks the prompt unit by unit (J/Tokenizer.java:110-127: a character outside the basic plane is two
// surrogates, each looked up on its own and then encoded as '?'), the sorted vocabulary is ordered as
// String.compareTo orders it, and the binary search takes the same probes as Arrays.binarySearch.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/llama2j_hip.h"
#include "host_internal.h"

namespace {

int fail(int code, const std::string &msg)
{
    l2j_set_error_(msg.c_str());
    return code;
}

typedef std::u16string jstring;  // a Java String: UTF-16 code units

// new String(bytes, UTF_8) for well-formed input; false for anything else (the reference would substitute
// U+FFFD; no tokenizer file or prompt in use holds such bytes).
bool utf8_to_jstring(const uint8_t *s, size_t n, jstring &out)
{
    out.clear();
    size_t i = 0;
    while (i < n) {
        uint32_t c = s[i];
        int more = 0;
        if (c < 0x80) more = 0;
        else if (c >= 0xC2 && c <= 0xDF) { more = 1; c &= 0x1F; }
        else if (c >= 0xE0 && c <= 0xEF) { more = 2; c &= 0x0F; }
        else if (c >= 0xF0 && c <= 0xF4) { more = 3; c &= 0x07; }
        else return false;
        if (i + more >= n && more) return false;
        for (int k = 1; k <= more; k++) {
            const uint32_t t = s[i + k];
            if ((t & 0xC0) != 0x80) return false;
            c = (c << 6) | (t & 0x3F);
        }
        if ((more == 2 && (c < 0x800 || (c >= 0xD800 && c <= 0xDFFF))) || (more == 3 && (c < 0x10000 || c > 0x10FFFF))) return false;
        if (c >= 0x10000) {
            c -= 0x10000;
            out.push_back((char16_t)(0xD800 + (c >> 10)));
            out.push_back((char16_t)(0xDC00 + (c & 0x3FF)));
        } else {
            out.push_back((char16_t)c);
        }
        i += 1 + more;
    }
    return true;
}

void append_utf8(std::string &out, uint32_t c)
{
    if (c < 0x80) out.push_back((char)c);
    else if (c < 0x800) { out.push_back((char)(0xC0 | (c >> 6))); out.push_back((char)(0x80 | (c & 0x3F))); }
    else if (c < 0x10000) {
        out.push_back((char)(0xE0 | (c >> 12))); out.push_back((char)(0x80 | ((c >> 6) & 0x3F))); out.push_back((char)(0x80 | (c & 0x3F)));
    } else {
        out.push_back((char)(0xF0 | (c >> 18))); out.push_back((char)(0x80 | ((c >> 12) & 0x3F)));
        out.push_back((char)(0x80 | ((c >> 6) & 0x3F))); out.push_back((char)(0x80 | (c & 0x3F)));
    }
}

// String.getBytes(UTF_8): surrogate pairs become one four-byte sequence, an unpaired surrogate becomes '?'
std::string jstring_to_utf8(const jstring &s)
{
    std::string out;
    for (size_t i = 0; i < s.size(); i++) {
        uint32_t c = s[i];
        if (c >= 0xD800 && c <= 0xDBFF && i + 1 < s.size() && s[i + 1] >= 0xDC00 && s[i + 1] <= 0xDFFF) {
            c = 0x10000 + ((c - 0xD800) << 10) + (s[i + 1] - 0xDC00);
            i++;
        } else if (c >= 0xD800 && c <= 0xDFFF) {
            c = '?';
        }
        append_utf8(out, c);
    }
    return out;
}

}  // namespace

struct l2j_tokenizer {
    std::vector<jstring> vocab;          // J/Tokenizer.java:22
    std::vector<float> scores;           // :23
    std::vector<int32_t> sorted;         // :25, 85: ids ordered by string
    std::vector<int32_t> first_single;   // first id whose string is exactly this one UTF-16 unit (:92-100), or -1

    // Arrays.binarySearch(sorted_vocab, key) with TokenIndex.compareTo (:27-31, 47-56)
    int lookup(const jstring &key) const
    {
        int low = 0, high = (int)sorted.size() - 1;
        while (low <= high) {
            const int mid = (int)(((unsigned)low + (unsigned)high) >> 1);
            const int cmp = vocab[sorted[mid]].compare(key);
            if (cmp < 0) low = mid + 1;
            else if (cmp > 0) high = mid - 1;
            else return sorted[mid];
        }
        return -1;
    }
};

extern "C" {

int l2j_tokenizer_open(const char *path, int32_t vocab_size, l2j_tokenizer **out)
{
    if (!path || !out || vocab_size <= 0) return fail(L2J_E_ARG, "bad argument");
    *out = nullptr;
    FILE *f = fopen(path, "rb");
    if (!f) return fail(L2J_E_IO, std::string("Cannot read tokenizer file ") + path);
    l2j_tokenizer *t = new l2j_tokenizer;
    t->vocab.resize(vocab_size);
    t->scores.resize(vocab_size);
    int32_t max_len_ignored = 0;
    bool ok = fread(&max_len_ignored, 4, 1, f) == 1;   // J/Tokenizer.java:70
    std::vector<uint8_t> buf;
    for (int i = 0; ok && i < vocab_size; i++) {
        int32_t len = 0;
        ok = fread(&t->scores[i], 4, 1, f) == 1 && fread(&len, 4, 1, f) == 1 && len >= 0 && len < (1 << 20);
        if (!ok) break;
        buf.resize((size_t)len);
        ok = len == 0 || fread(buf.data(), 1, (size_t)len, f) == (size_t)len;
        if (ok && !utf8_to_jstring(buf.data(), buf.size(), t->vocab[i])) {
            fclose(f);
            delete t;
            return fail(L2J_E_IO, "tokenizer file: token " + std::to_string(i) + " is not UTF-8");
        }
    }
    fclose(f);
    if (!ok) {
        delete t;
        return fail(L2J_E_IO, std::string("Cannot read tokenizer file ") + path);
    }
    t->sorted.resize(vocab_size);
    for (int i = 0; i < vocab_size; i++) t->sorted[i] = i;
    std::stable_sort(t->sorted.begin(), t->sorted.end(),
                     [&](int32_t a, int32_t b) { return t->vocab[a].compare(t->vocab[b]) < 0; });  // :85
    t->first_single.assign(65536, -1);
    for (int i = vocab_size - 1; i >= 0; i--)
        if (t->vocab[i].size() == 1) t->first_single[t->vocab[i][0]] = i;
    *out = t;
    return L2J_OK;
}

void l2j_tokenizer_close(l2j_tokenizer *t) { delete t; }

int l2j_bpe_encode(l2j_tokenizer *t, const char *prompt_utf8, int32_t *tokens, int32_t cap, int32_t *n_out)
{
    if (!t || !prompt_utf8 || !tokens || !n_out) return fail(L2J_E_ARG, "null argument");
    jstring prompt;
    if (!utf8_to_jstring((const uint8_t *)prompt_utf8, strlen(prompt_utf8), prompt)) return fail(L2J_E_ARG, "prompt is not UTF-8");
    std::vector<int32_t> tok;
    tok.reserve(prompt.size() * 2 + 1);
    tok.push_back(t->lookup(jstring(1, u' ')));  // add_dummy_prefix (:107)
    for (char16_t c : prompt) {
        const int id = t->first_single[c];
        if (id != -1) {
            tok.push_back(id);
        } else {
            // byte fallback (:118-125): the bytes are Java's signed bytes, so those above 0x7f give negative ids
            const std::string bytes = jstring_to_utf8(jstring(1, c));
            for (char b : bytes) tok.push_back((int32_t)(int8_t)b + 3);
        }
    }
    const int V = (int)t->vocab.size();
    while (true) {  // merge the best consecutive pair (:130-159)
        float best_score = -1e10f;
        int best_id = -1, best_idx = -1;
        for (int i = 0; i + 1 < (int)tok.size(); i++) {
            if (tok[i] < 0 || tok[i] >= V || tok[i + 1] < 0 || tok[i + 1] >= V)
                return fail(L2J_E_ARG, "bpe_encode: token id " + std::to_string(tok[i] < 0 || tok[i] >= V ? tok[i] : tok[i + 1]) +
                                           " outside the vocabulary (ArrayIndexOutOfBoundsException in the reference: no ' ' token, "
                                           "or a character missing from the vocabulary whose UTF-8 bytes are above 0x7f)");
            const int id = t->lookup(t->vocab[tok[i]] + t->vocab[tok[i + 1]]);
            if (id != -1 && t->scores[id] > best_score) {
                best_score = t->scores[id];
                best_id = id;
                best_idx = i;
            }
        }
        if (best_idx == -1) break;
        tok[best_idx] = best_id;
        tok.erase(tok.begin() + best_idx + 1);
    }
    *n_out = (int32_t)tok.size();
    if ((int)tok.size() > cap) return fail(L2J_E_SIZE, "bpe_encode: output buffer too small");
    memcpy(tokens, tok.data(), tok.size() * sizeof(int32_t));
    return L2J_OK;
}

int l2j_bpe_decode(l2j_tokenizer *t, int32_t token, int32_t next, char *out_utf8, int32_t cap, int32_t *len_out)
{
    if (!t || !out_utf8 || !len_out || cap <= 0) return fail(L2J_E_ARG, "null argument");
    if (next < 0 || next >= (int)t->vocab.size()) return fail(L2J_E_ARG, "bpe_decode: token id outside the vocabulary");
    const jstring &piece = t->vocab[next];
    jstring s = piece;
    if (token == 1) {  // after BOS a leading blank is stripped (:191)
        if (piece.empty()) return fail(L2J_E_ARG, "bpe_decode: empty token after BOS (StringIndexOutOfBoundsException in the reference)");
        if (piece[0] == u' ') s = piece.substr(1);
    }
    *len_out = -1;  // null
    // "<0x([\da-fA-F]*)>" (:187, 194-206)
    bool raw = s.size() >= 4 && s[0] == u'<' && s[1] == u'0' && s[2] == u'x' && s.back() == u'>';
    for (size_t i = 3; raw && i + 1 < s.size(); i++) {
        const char16_t c = s[i];
        raw = (c >= u'0' && c <= u'9') || (c >= u'a' && c <= u'f') || (c >= u'A' && c <= u'F');
    }
    std::string out;
    if (raw) {
        if (s.size() == 4) { out_utf8[0] = 0; return L2J_OK; }  // Integer.parseInt("") throws: null
        uint64_t value = 0;
        for (size_t i = 3; i + 1 < s.size(); i++) {
            const char16_t c = s[i];
            value = value * 16 + (c <= u'9' ? c - u'0' : (c | 0x20) - u'a' + 10);
            if (value > 0x7FFFFFFFull) { out_utf8[0] = 0; return L2J_OK; }  // NumberFormatException: null
        }
        const uint32_t c = (uint32_t)value & 0xFF;
        const bool iso_control = c <= 0x1F || (c >= 0x7F && c <= 0x9F);  // Character.isISOControl
        if (c != '\n' && iso_control) { out_utf8[0] = 0; return L2J_OK; }
        append_utf8(out, c);   // Character.toString((char) c): a Latin-1 character, not a raw byte
    } else {
        out = jstring_to_utf8(s);
    }
    if ((int)out.size() + 1 > cap) return fail(L2J_E_SIZE, "bpe_decode: output buffer too small");
    memcpy(out_utf8, out.data(), out.size());
    out_utf8[out.size()] = 0;
    *len_out = (int32_t)out.size();
    return L2J_OK;
}

}  // extern "C"
