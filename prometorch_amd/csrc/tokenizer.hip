// Text <-> token ids on the host: the tokenizer that sits in front of the prompt path and behind the sampler.
//
// Counterpart of GGUFTokenizer (torch/io/tokenizer.h:24-643) and of GGUFModel::apply_chat_template
// (torch/io/gguf_model.h:4178-4236).  Same results, own construction: one byte classifier drives the GPT-2 style
// splitter, the byte -> code-point alphabet is a 256-entry table built once, a merge's key is the merge string itself.
// Behaviour kept from the reference, including its corners:
//   * vocabulary strings that look like <...> (but not <0xNN>-like: longer than 4 bytes or second byte != '0') are
//     special tokens, matched longest first before any other processing (tokenizer.h:100-114, :193-229);
//   * model "gpt2": contractions 's 't 'm 'd 're 've 'll; one optional leading white-space byte glued to the next
//     run; runs of letters (ASCII letters and every byte >= 0xC2, continuation bytes included), of ASCII digits, of
//     anything else; white-space runs keep their last byte for the next word unless the text ends (:260-366); every
//     word is mapped byte -> code point (GPT-2 bytes_to_unicode, :375-396), looked up whole, else merged (:397-409);
//   * any other model: white space is dropped except '\n', a U+2581 marks the start of every word, and the whole
//     segment is ONE piece for the merges (:238-258);
//   * merges: lowest rank first, leftmost on ties, until none applies; unknown symbols fall back to <0xNN> per byte,
//     then to the unknown id (:414-457, :513-529);
//   * no merges at all: greedy longest match of at most 64 bytes (:463-507);
//   * decoding a token: <0xNN> is that byte; U+2581, U+0120 -> ' ', U+010A -> '\n', U+0109 -> '\t'; remaining
//     code points of the GPT-2 byte alphabet go back to their byte (:535-630).
#include "ptm_common.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

struct ptm_tokenizer {
    std::vector<std::string> vocab;
    std::unordered_map<std::string, int32_t> token_to_id;   // a string listed twice keeps its LAST id (tokenizer.h:55-57)
    std::unordered_map<std::string, int32_t> merge_rank;    // "left right" -> rank; listed twice: last rank (:96-98)
    size_t n_merges = 0;
    std::vector<std::pair<std::string, int32_t>> specials;  // longest first
    int32_t bos = 1, eos = 2, pad = -1, unk = 0;
    bool add_bos = true;
    bool gpt2 = false;
    std::string byte_cp[256];  // GPT-2 alphabet: byte -> UTF-8 of its code point
};

namespace ptm {

static const char kWordMark[] = "\xe2\x96\x81";  // U+2581

static size_t utf8_len(unsigned char c) {
    if ((c & 0x80) == 0) return 1;
    if ((c & 0xE0) == 0xC0) return 2;
    if ((c & 0xF0) == 0xE0) return 3;
    if ((c & 0xF8) == 0xF0) return 4;
    return 1;
}

static int byte_to_cp(int b) {
    if ((b >= 33 && b <= 126) || (b >= 161 && b <= 172) || (b >= 174 && b <= 255)) return b;
    if (b <= 32) return 0x100 + b;
    if (b >= 127 && b <= 160) return 0x121 + (b - 127);
    return 0x143;  // 173
}
static int cp_to_byte(uint32_t cp) {  // -1: not a code point of the byte alphabet that decoding maps back
    if ((cp >= 161 && cp <= 172) || (cp >= 174 && cp <= 255)) return (int)cp;
    if (cp >= 0x100 && cp <= 0x120) return (int)(cp - 0x100);
    if (cp >= 0x121 && cp <= 0x142) return (int)(127 + (cp - 0x121));
    if (cp == 0x143) return 173;
    return -1;
}
static void append_cp(std::string& dst, int cp) {
    if (cp < 0x80) {
        dst += (char)cp;
    } else if (cp < 0x800) {
        dst += (char)(0xC0 | (cp >> 6));
        dst += (char)(0x80 | (cp & 0x3F));
    } else {
        dst += (char)(0xE0 | (cp >> 12));
        dst += (char)(0x80 | ((cp >> 6) & 0x3F));
        dst += (char)(0x80 | (cp & 0x3F));
    }
}

static void finish_tables(ptm_tokenizer* t) {
    for (size_t i = 0; i < t->vocab.size(); ++i) t->token_to_id[t->vocab[i]] = (int32_t)i;
    for (size_t i = 0; i < t->vocab.size(); ++i) {
        const std::string& tok = t->vocab[i];
        if (tok.size() >= 3 && tok[0] == '<' && tok.back() == '>' && (tok.size() > 4 || tok[1] != '0'))
            t->specials.push_back({tok, (int32_t)i});
    }
    // longest first; equal lengths keep vocabulary order (two different strings of one length never match at one place)
    std::stable_sort(t->specials.begin(), t->specials.end(),
                     [](const auto& a, const auto& b) { return a.first.size() > b.first.size(); });
    for (int b = 0; b < 256; ++b) append_cp(t->byte_cp[b], byte_to_cp(b));
}

static void add_merge(ptm_tokenizer* t, const std::string& m) {
    if (m.find(' ') == std::string::npos) return;  // not "left right": not a merge, and it takes no rank (:74-80)
    t->merge_rank[m] = (int32_t)t->n_merges++;      // left + " " + right is the string itself
}

static void byte_fallback(const ptm_tokenizer* t, uint8_t b, std::vector<int32_t>& out) {
    char buf[8];
    snprintf(buf, sizeof(buf), "<0x%02X>", b);
    auto it = t->token_to_id.find(buf);
    out.push_back(it != t->token_to_id.end() ? it->second : t->unk);
}

// merges over one piece
static void bpe_piece(const ptm_tokenizer* t, const std::string& piece, std::vector<int32_t>& out) {
    std::vector<std::string> sym;
    for (size_t i = 0; i < piece.size();) {
        size_t n = utf8_len((unsigned char)piece[i]);
        if (i + n > piece.size()) n = 1;
        sym.emplace_back(piece, i, n);
        i += n;
    }
    std::string key;
    while (sym.size() >= 2) {
        int32_t best = INT32_MAX;
        size_t at = SIZE_MAX;
        for (size_t j = 0; j + 1 < sym.size(); ++j) {
            key.assign(sym[j]).append(1, ' ').append(sym[j + 1]);
            auto it = t->merge_rank.find(key);
            if (it != t->merge_rank.end() && it->second < best) { best = it->second; at = j; }
        }
        if (at == SIZE_MAX) break;
        sym[at] += sym[at + 1];
        sym.erase(sym.begin() + (long)at + 1);
    }
    for (const std::string& s : sym) {
        auto it = t->token_to_id.find(s);
        if (it != t->token_to_id.end()) out.push_back(it->second);
        else for (unsigned char c : s) byte_fallback(t, c, out);
    }
}

// byte classes of the GPT-2 style splitter
enum : uint8_t { C_OTHER, C_SPACE, C_DIGIT, C_LETTER, C_CONT };
static uint8_t byte_class(unsigned char c) {
    if (c == ' ' || c == '\t' || c == '\n' || c == '\r' || c == '\v' || c == '\f') return C_SPACE;
    if (c >= '0' && c <= '9') return C_DIGIT;
    if ((c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || c >= 0xC2) return C_LETTER;
    if (c >= 0x80 && c <= 0xBF) return C_CONT;
    return C_OTHER;  // ASCII punctuation and control bytes, 0xC0, 0xC1
}

static size_t contraction_len(const std::string& s, size_t i) {
    if (i >= s.size() || s[i] != '\'' || i + 1 >= s.size()) return 0;
    const char b = s[i + 1];
    if (b == 's' || b == 't' || b == 'm' || b == 'd') return 2;
    if (i + 2 < s.size()) {
        const char c = s[i + 2];
        if ((b == 'r' && c == 'e') || (b == 'v' && c == 'e') || (b == 'l' && c == 'l')) return 3;
    }
    return 0;
}

// The reference's scanner (tokenizer.h:302-366).  One difference, on purpose: a continuation byte (0x80..0xBF) that
// does not follow a letter makes the reference emit empty words for ever (its symbol run stops AT the byte without
// consuming it); here such a byte is a word of its own (with the white-space byte glued in front, if any).
static void split_gpt2(const std::string& s, std::vector<std::string>& words) {
    const size_t N = s.size();
    size_t i = 0;
    while (i < N) {
        if (const size_t n = contraction_len(s, i)) { words.emplace_back(s, i, n); i += n; continue; }
        const size_t start = i;
        if (byte_class((unsigned char)s[i]) == C_SPACE) {
            if (i + 1 >= N || byte_class((unsigned char)s[i + 1]) == C_SPACE) {
                // a run of white space: all of it at the end of the text, otherwise all but its last byte,
                // which is glued to the word that follows
                size_t e = i;
                while (e < N && byte_class((unsigned char)s[e]) == C_SPACE) ++e;
                const size_t end = e == N ? e : e - 1;
                words.emplace_back(s, start, end - start);
                i = end;
                continue;
            }
            ++i;  // one white-space byte glued to what follows
        }
        switch (byte_class((unsigned char)s[i])) {
            case C_LETTER:
                while (i < N) { const uint8_t c = byte_class((unsigned char)s[i]); if (c != C_LETTER && c != C_CONT) break; ++i; }
                break;
            case C_DIGIT:
                while (i < N && byte_class((unsigned char)s[i]) == C_DIGIT) ++i;
                break;
            case C_OTHER:
                while (i < N && byte_class((unsigned char)s[i]) == C_OTHER) ++i;
                break;
            default:  // stray continuation byte
                ++i;
                break;
        }
        words.emplace_back(s, start, i - start);
    }
}

static void encode_bpe(const ptm_tokenizer* t, const std::string& text, std::vector<int32_t>& out) {
    if (!t->gpt2) {
        std::string piece;
        bool at_start = true;
        for (char c : text) {
            if (c == ' ' || c == '\n' || c == '\t') {
                at_start = true;
                if (c == '\n') piece += c;
                continue;
            }
            if (at_start) { piece += kWordMark; at_start = false; }
            piece += c;
        }
        if (!piece.empty()) bpe_piece(t, piece, out);
        return;
    }
    std::vector<std::string> words;
    split_gpt2(text, words);
    std::string w;
    for (const std::string& word : words) {
        w.clear();
        for (unsigned char c : word) w += t->byte_cp[c];
        auto it = t->token_to_id.find(w);
        if (it != t->token_to_id.end()) out.push_back(it->second);
        else bpe_piece(t, w, out);
    }
}

static void encode_greedy(const ptm_tokenizer* t, const std::string& text, std::vector<int32_t>& out) {
    std::string p;
    bool at_start = true;
    for (char c : text) {
        if (c == ' ') { at_start = true; continue; }
        if (at_start) { p += kWordMark; at_start = false; }
        p += c;
    }
    for (size_t i = 0; i < p.size();) {
        size_t len = std::min(p.size() - i, (size_t)64), hit = 0;
        int32_t id = t->unk;
        for (; len >= 1; --len) {
            auto it = t->token_to_id.find(p.substr(i, len));
            if (it != t->token_to_id.end()) { id = it->second; hit = len; break; }
        }
        if (hit) { out.push_back(id); i += hit; }
        else { byte_fallback(t, (uint8_t)p[i], out); i += 1; }
    }
}

static void encode_text(const ptm_tokenizer* t, const std::string& text, bool use_bos, std::vector<int32_t>& out) {
    if (use_bos && t->add_bos && t->bos >= 0) out.push_back(t->bos);
    if (text.empty()) return;
    auto plain = [&](const std::string& seg) {
        if (seg.empty()) return;
        if (t->n_merges) encode_bpe(t, seg, out);
        else encode_greedy(t, seg, out);
    };
    if (t->specials.empty()) { plain(text); return; }
    size_t pos = 0;
    while (pos < text.size()) {
        bool matched = false;
        for (const auto& sp : t->specials)
            if (text.compare(pos, sp.first.size(), sp.first) == 0) {
                out.push_back(sp.second);
                pos += sp.first.size();
                matched = true;
                break;
            }
        if (matched) continue;
        size_t next = text.size();
        for (const auto& sp : t->specials) {
            const size_t p = text.find(sp.first, pos);
            if (p != std::string::npos && p < next) next = p;
        }
        plain(text.substr(pos, next - pos));
        pos = next;
    }
}

static int hexval(char c) {
    if (c >= '0' && c <= '9') return c - '0';
    if (c >= 'a' && c <= 'f') return c - 'a' + 10;
    if (c >= 'A' && c <= 'F') return c - 'A' + 10;
    return -1;
}

static void replace_all(std::string& s, const char* what, size_t n, char with) {
    for (size_t pos = 0; (pos = s.find(what, pos, n)) != std::string::npos; pos += 1) s.replace(pos, n, 1, with);
}

static void decode_token_str(const std::string& token, std::string& out) {
    if (token.size() == 6 && token[0] == '<' && token[1] == '0' && token[2] == 'x' && token[5] == '>' &&
        hexval(token[3]) >= 0 && hexval(token[4]) >= 0) {
        out += (char)(hexval(token[3]) * 16 + hexval(token[4]));
        return;
    }
    std::string r = token;
    replace_all(r, kWordMark, 3, ' ');
    replace_all(r, "\xc4\xa0", 2, ' ');
    replace_all(r, "\xc4\x8a", 2, '\n');
    replace_all(r, "\xc4\x89", 2, '\t');
    for (size_t i = 0; i < r.size();) {
        const unsigned char c = (unsigned char)r[i];
        const size_t n = utf8_len(c);
        if (n == 1 || i + n > r.size()) { out += r[i]; ++i; continue; }
        uint32_t cp = 0;
        if (n == 2) cp = ((c & 0x1Fu) << 6) | ((unsigned char)r[i + 1] & 0x3Fu);
        else if (n == 3) cp = ((c & 0x0Fu) << 12) | (((unsigned char)r[i + 1] & 0x3Fu) << 6) | ((unsigned char)r[i + 2] & 0x3Fu);
        else cp = ((c & 0x07u) << 18) | (((unsigned char)r[i + 1] & 0x3Fu) << 12) | (((unsigned char)r[i + 2] & 0x3Fu) << 6) |
                  ((unsigned char)r[i + 3] & 0x3Fu);
        const int b = cp_to_byte(cp);
        if (b >= 0) out += (char)b;
        else out.append(r, i, n);
        i += n;
    }
}

static int copy_out(const std::string& s, char* out, int64_t cap, int64_t* len) {
    if (len) *len = (int64_t)s.size();
    if ((int64_t)s.size() > cap) return PTM_E_RANGE;
    if (!s.empty()) memcpy(out, s.data(), s.size());
    return PTM_OK;
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int ptm_tokenizer_create(const char* const* tokens, const int32_t* token_lens, int32_t n_tokens, const char* const* merges,
                         const int32_t* merge_lens, int32_t n_merges, const char* model_type, int32_t bos_id, int32_t eos_id,
                         int32_t pad_id, int32_t unk_id, int add_bos, ptm_tokenizer** out) {
    if (!out || (n_tokens > 0 && (!tokens || !token_lens)) || (n_merges > 0 && (!merges || !merge_lens))) return PTM_E_NULL;
    if (n_tokens < 0 || n_merges < 0) return PTM_E_SHAPE;
    ptm_tokenizer* t = new ptm_tokenizer();
    t->vocab.reserve((size_t)n_tokens);
    for (int32_t i = 0; i < n_tokens; ++i) {
        if (!tokens[i] || token_lens[i] < 0) { delete t; return PTM_E_NULL; }
        t->vocab.emplace_back(tokens[i], (size_t)token_lens[i]);
    }
    for (int32_t i = 0; i < n_merges; ++i) {
        if (!merges[i] || merge_lens[i] < 0) { delete t; return PTM_E_NULL; }
        add_merge(t, std::string(merges[i], (size_t)merge_lens[i]));
    }
    t->gpt2 = model_type && strcmp(model_type, "gpt2") == 0;
    t->bos = bos_id; t->eos = eos_id; t->pad = pad_id; t->unk = unk_id;
    t->add_bos = add_bos != 0;
    finish_tables(t);
    *out = t;
    return PTM_OK;
}

// tokenizer.ggml.{model, tokens, merges, bos_token_id, eos_token_id, padding_token_id, unknown_token_id, add_bos_token}
// (tokenizer.h:42-93; defaults: model "llama", ids 1 / 2 / -1 / 0, add_bos true)
int ptm_tokenizer_from_gguf(const ptm_gguf* g, ptm_tokenizer** out) {
    if (!g || !out) return PTM_E_NULL;
    ptm_tokenizer* t = new ptm_tokenizer();
    const char* model = ptm_gguf_get_string(g, "tokenizer.ggml.model");
    t->gpt2 = model && strcmp(model, "gpt2") == 0;
    uint32_t et = 0;
    int64_t n = 0;
    if (ptm_gguf_get_array(g, "tokenizer.ggml.tokens", &et, &n) == PTM_OK) {
        if (et != 8) { delete t; return PTM_E_FORMAT; }
        t->vocab.reserve((size_t)n);
        for (int64_t i = 0; i < n; ++i) {
            const char* p; int64_t len;
            if (ptm_gguf_array_string(g, "tokenizer.ggml.tokens", i, &p, &len) != PTM_OK) { delete t; return PTM_E_FORMAT; }
            t->vocab.emplace_back(p, (size_t)len);
        }
    }
    if (ptm_gguf_get_array(g, "tokenizer.ggml.merges", &et, &n) == PTM_OK) {
        if (et != 8) { delete t; return PTM_E_FORMAT; }
        for (int64_t i = 0; i < n; ++i) {
            const char* p; int64_t len;
            if (ptm_gguf_array_string(g, "tokenizer.ggml.merges", i, &p, &len) != PTM_OK) { delete t; return PTM_E_FORMAT; }
            add_merge(t, std::string(p, (size_t)len));
        }
    }
    int64_t v;
    if (ptm_gguf_get_int(g, "tokenizer.ggml.bos_token_id", &v) == PTM_OK) t->bos = (int32_t)v;
    if (ptm_gguf_get_int(g, "tokenizer.ggml.eos_token_id", &v) == PTM_OK) t->eos = (int32_t)v;
    if (ptm_gguf_get_int(g, "tokenizer.ggml.padding_token_id", &v) == PTM_OK) t->pad = (int32_t)v;
    if (ptm_gguf_get_int(g, "tokenizer.ggml.unknown_token_id", &v) == PTM_OK) t->unk = (int32_t)v;
    if (ptm_gguf_get_int(g, "tokenizer.ggml.add_bos_token", &v) == PTM_OK) t->add_bos = v != 0;
    finish_tables(t);
    *out = t;
    return PTM_OK;
}

void ptm_tokenizer_free(ptm_tokenizer* t) { delete t; }

int32_t ptm_tokenizer_vocab_size(const ptm_tokenizer* t) { return t ? (int32_t)t->vocab.size() : 0; }

int ptm_tokenizer_special_ids(const ptm_tokenizer* t, int32_t* bos, int32_t* eos, int32_t* pad, int32_t* unk) {
    if (!t) return PTM_E_NULL;
    if (bos) *bos = t->bos;
    if (eos) *eos = t->eos;
    if (pad) *pad = t->pad;
    if (unk) *unk = t->unk;
    return PTM_OK;
}

int ptm_tokenizer_encode(const ptm_tokenizer* t, const char* text, int64_t text_len, int use_bos, int32_t* ids, int64_t cap,
                         int64_t* n_ids) {
    if (!t || (!text && text_len > 0) || !n_ids || (!ids && cap > 0)) return PTM_E_NULL;
    if (text_len < 0 || cap < 0) return PTM_E_SHAPE;
    std::vector<int32_t> out;
    encode_text(t, std::string(text ? text : "", (size_t)text_len), use_bos != 0, out);
    *n_ids = (int64_t)out.size();
    if ((int64_t)out.size() > cap) return PTM_E_RANGE;
    if (!out.empty()) memcpy(ids, out.data(), out.size() * sizeof(int32_t));
    return PTM_OK;
}

int ptm_tokenizer_decode(const ptm_tokenizer* t, const int32_t* ids, int64_t n_ids, int skip_special, char* out, int64_t cap,
                         int64_t* len) {
    if (!t || (!ids && n_ids > 0) || (!out && cap > 0)) return PTM_E_NULL;
    if (n_ids < 0 || cap < 0) return PTM_E_SHAPE;
    std::string s;
    for (int64_t i = 0; i < n_ids; ++i) {
        const int32_t id = ids[i];
        if (skip_special && (id == t->bos || id == t->eos || id == t->pad)) continue;
        if (id >= 0 && id < (int32_t)t->vocab.size()) decode_token_str(t->vocab[(size_t)id], s);
    }
    return copy_out(s, out, cap, len);
}

int ptm_tokenizer_token(const ptm_tokenizer* t, int32_t id, char* out, int64_t cap, int64_t* len) {
    if (!t || (!out && cap > 0)) return PTM_E_NULL;
    std::string s;
    if (id >= 0 && id < (int32_t)t->vocab.size()) decode_token_str(t->vocab[(size_t)id], s);
    return copy_out(s, out, cap, len);
}

// apply_chat_template (gguf_model.h:4178-4236).  The reference takes the system prompt and the no-think switch from the
// environment (PT_SYSTEM_PROMPT, PT_NO_THINK); here they are arguments: system NULL = its default text, "" = none.
int ptm_chat_template(const char* architecture, const char* model_name, const char* system, int no_think, const char* prompt,
                      char* out, int64_t cap, int64_t* len) {
    if (!architecture || !prompt || (!out && cap > 0)) return PTM_E_NULL;
    const std::string arch = architecture, user = prompt;
    const std::string sys = system ? system : "You are a helpful assistant.";
    std::string r;
    if (arch == "qwen3" || arch == "qwen2") {
        if (no_think && arch == "qwen3") r = "<|im_start|>system\n" + (sys.empty() ? std::string("/no_think") : sys + "\n/no_think") + "<|im_end|>\n";
        else if (!sys.empty()) r = "<|im_start|>system\n" + sys + "<|im_end|>\n";
        r += "<|im_start|>user\n" + user + "<|im_end|>\n<|im_start|>assistant\n";
    } else if (arch == "phi3" || arch == "phi2") {
        if (!sys.empty()) r = "<|system|>\n" + sys + "<|end|>\n";
        r += "<|user|>\n" + user + "<|end|>\n<|assistant|>\n";
    } else if (arch == "gemma3" || arch == "gemma2") {
        r = "<start_of_turn>user\n" + (sys.empty() ? user : sys + "\n\n" + user) + "<end_of_turn>\n<start_of_turn>model\n";
    } else if (arch == "llama") {
        std::string lname = model_name ? model_name : "";
        for (char& c : lname) if (c >= 'A' && c <= 'Z') c = (char)(c + 32);
        if (lname.find("mistral") != std::string::npos) {
            r = sys.empty() ? "<s>[INST] " + user + " [/INST]" : "<s>[INST] <<SYS>>\n" + sys + "\n<</SYS>>\n\n" + user + " [/INST]";
        } else {
            r = "<|begin_of_text|>";
            if (!sys.empty()) r += "<|start_header_id|>system<|end_header_id|>\n\n" + sys + "<|eot_id|>";
            r += "<|start_header_id|>user<|end_header_id|>\n\n" + user + "<|eot_id|><|start_header_id|>assistant<|end_header_id|>\n\n";
        }
    } else {
        r = user;
    }
    return copy_out(r, out, cap, len);
}

}  // extern "C"
