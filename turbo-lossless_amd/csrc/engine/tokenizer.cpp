// The two tokenizer backends behind the reference's engine/tokenizer.h API (see include/turbo/tokenizer.h):
// sentencepiece BPE models (sp_model.cpp) and byte-level BPE tables (this file).  Host code only.
#include "turbo/tokenizer.h"

#include "sp_model.h"

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <fstream>
#include <iterator>
#include <unordered_map>

namespace {

struct Merge {
    int left, right, result;   // symbol numbers
    int next_same;             // next rank that lists the same (left, right) pair, -1 = none
};

struct BpeModel {
    // vocabulary as the reference keeps it (engine/tokenizer.cpp:32-39,171-173): the last id of a repeated
    // string wins for encoding, every id keeps its own string for decoding
    std::vector<std::string> id_to_token;
    std::unordered_map<std::string, int> token_to_id;
    std::string byte_encoder[256];
    std::unordered_map<std::string, uint8_t> byte_decoder;
    // symbols = every string encoding can meet: byte-encoder outputs, merge parts, merge results
    std::unordered_map<std::string, int> symbol_of;
    std::vector<int> symbol_id;            // symbol -> vocabulary id, 0 when not in the vocabulary (tokenizer.cpp:321-323)
    int byte_symbol[256];
    std::vector<Merge> merges;             // by rank
    std::unordered_map<uint64_t, int> first_rank;   // (left << 32 | right) -> lowest rank of that pair

    int intern(const std::string& s)
    {
        auto it = symbol_of.find(s);
        if (it != symbol_of.end()) return it->second;
        const int n = (int)symbol_id.size();
        symbol_of.emplace(s, n);
        auto v = token_to_id.find(s);
        symbol_id.push_back(v == token_to_id.end() ? 0 : v->second);
        return n;
    }
    // lowest rank above `after` at which the pair (l, r) is listed, -1 = none
    int rank_after(int l, int r, int after) const
    {
        auto it = first_rank.find(((uint64_t)(uint32_t)l << 32) | (uint32_t)r);
        if (it == first_rank.end()) return -1;
        int rank = it->second;
        while (rank >= 0 && rank <= after) rank = merges[rank].next_same;
        return rank;
    }
};

bool read_exact(std::ifstream& f, void* dst, size_t n) { return (bool)f.read((char*)dst, (std::streamsize)n); }

bool read_string(std::ifstream& f, size_t n, std::string* s)
{
    s->assign(n, '\0');
    return n == 0 || read_exact(f, &(*s)[0], n);
}

BpeModel* load_bpe(const std::string& dir, int* bos, int* eos)
{
    std::ifstream vf(dir + "/vocab.bin", std::ios::binary), mf(dir + "/merges.bin", std::ios::binary);
    if (!vf || !mf) return nullptr;
    auto* m = new BpeModel();
    auto fail = [&](const char* what) {
        fprintf(stderr, "tokenizer: %s in %s\n", what, dir.c_str());
        delete m;
        return (BpeModel*)nullptr;
    };
    int32_t n_vocab = 0, b = 0, e = 0;
    if (!read_exact(vf, &n_vocab, 4) || !read_exact(vf, &b, 4) || !read_exact(vf, &e, 4) || n_vocab < 0)
        return fail("vocab.bin has no header");
    *bos = b;
    *eos = e;
    m->id_to_token.resize((size_t)n_vocab);
    for (int i = 0; i < n_vocab; i++) {
        uint16_t len;
        if (!read_exact(vf, &len, 2) || !read_string(vf, len, &m->id_to_token[i])) return fail("vocab.bin is truncated");
        m->token_to_id[m->id_to_token[i]] = i;
    }
    std::ifstream bf(dir + "/byte_encoder.bin", std::ios::binary);
    for (int i = 0; i < 256; i++) {
        if (bf) {
            uint8_t len;
            if (!read_exact(bf, &len, 1) || !read_string(bf, len, &m->byte_encoder[i]))
                return fail("byte_encoder.bin is truncated");
            if (len == 0) return fail("byte_encoder.bin maps a byte to the empty string");
        } else {
            m->byte_encoder[i] = std::string(1, (char)i);      // engine/tokenizer.cpp:195-198
        }
    }
    for (int i = 0; i < 256; i++) {
        m->byte_decoder[m->byte_encoder[i]] = (uint8_t)i;
        m->byte_symbol[i] = m->intern(m->byte_encoder[i]);
    }
    int32_t n_merges = 0;
    if (!read_exact(mf, &n_merges, 4) || n_merges < 0) return fail("merges.bin has no header");
    m->merges.reserve((size_t)n_merges);
    std::unordered_map<uint64_t, int> last_rank;
    std::string a, c;
    for (int r = 0; r < n_merges; r++) {
        uint16_t la, lb;
        if (!read_exact(mf, &la, 2) || !read_exact(mf, &lb, 2) || !read_string(mf, la, &a) || !read_string(mf, lb, &c))
            return fail("merges.bin is truncated");
        if (la == 0 || lb == 0) return fail("merges.bin lists a merge with an empty part");
        Merge g;
        g.left = m->intern(a);
        g.right = m->intern(c);
        g.result = m->intern(a + c);
        g.next_same = -1;
        const uint64_t key = ((uint64_t)(uint32_t)g.left << 32) | (uint32_t)g.right;
        auto it = last_rank.find(key);
        if (it == last_rank.end()) m->first_rank.emplace(key, r);
        else m->merges[it->second].next_same = r;
        last_rank[key] = r;
        m->merges.push_back(g);
    }
    return m;
}

// engine/tokenizer.cpp:295-326 in O(n log n).  Nodes are the text's bytes; a merge keeps the left node and
// drops the right one, so a node's index orders it within the text for good.  A candidate is an adjacent pair
// with the lowest rank its pair has above the rank that was current when the pair came to be (the reference's
// loop never returns to an earlier merge); candidates leave the queue by (rank, position), which is the
// order of the reference's nested loops, and are dropped when either node has changed since.
std::vector<int> bpe_encode(const BpeModel* m, const std::string& text)
{
    const int n = (int)text.size();
    std::vector<int> sym((size_t)n), next((size_t)n), prev((size_t)n);
    for (int i = 0; i < n; i++) {
        sym[i] = m->byte_symbol[(uint8_t)text[i]];
        prev[i] = i - 1;
        next[i] = i + 1 < n ? i + 1 : -1;
    }
    struct Cand {
        int rank, pos, l, r;
    };
    auto later = [](const Cand& x, const Cand& y) { return x.rank != y.rank ? x.rank > y.rank : x.pos > y.pos; };
    std::vector<Cand> heap;                    // binary heap, earliest (rank, position) on top
    heap.reserve((size_t)n);
    auto offer = [&](int i, int after, bool sift) {
        const int j = next[i];
        if (j < 0) return;
        const int rank = m->rank_after(sym[i], sym[j], after);
        if (rank < 0) return;
        heap.push_back({rank, i, sym[i], sym[j]});
        if (sift) std::push_heap(heap.begin(), heap.end(), later);
    };
    for (int i = 0; i + 1 < n; i++) offer(i, -1, false);
    std::make_heap(heap.begin(), heap.end(), later);
    while (!heap.empty()) {
        std::pop_heap(heap.begin(), heap.end(), later);
        const Cand c = heap.back();
        heap.pop_back();
        const int i = c.pos, j = next[i];
        if (sym[i] != c.l || j < 0 || sym[j] != c.r) continue;
        sym[i] = m->merges[c.rank].result;
        sym[j] = -1;
        next[i] = next[j];
        if (next[j] >= 0) prev[next[j]] = i;
        if (prev[i] >= 0) offer(prev[i], c.rank, true);
        offer(i, c.rank, true);
    }
    std::vector<int> ids;
    for (int i = n > 0 ? 0 : -1; i >= 0; i = next[i]) ids.push_back(m->symbol_id[sym[i]]);
    return ids;
}

std::vector<int> encode_plain(Tokenizer* tok, const std::string& text)
{
    if (tok->type == 0) return ((const SpModel*)tok->sp_model)->encode(text);
    return bpe_encode((const BpeModel*)tok->sp_model, text);
}

// engine/tokenizer.cpp:50-59: the integer after "key": in a JSON fragment, -1 when the key is absent
int json_int_after(const std::string& json, const std::string& key)
{
    size_t pos = json.find("\"" + key + "\"");
    if (pos == std::string::npos) return -1;
    pos = json.find(':', pos);
    if (pos == std::string::npos) return -1;
    pos++;
    while (pos < json.size() && (json[pos] == ' ' || json[pos] == '\t')) pos++;
    return atoi(json.c_str() + pos);
}

// engine/tokenizer.cpp:85-152, same reading of tokenizer.json, quirks included: every object of the "added_tokens"
// array that contains the text "special" (quoted) and the text true anywhere counts as special; its "content" is
// taken raw up to the next quote (no unescaping); ids <= 2 and one-character contents are left out; a content of
// </s> moves eos_id.
void load_special_tokens(Tokenizer* tok, const std::string& model_dir)
{
    std::ifstream f(model_dir + "/tokenizer.json");
    if (!f) return;
    const std::string json((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    const size_t added = json.find("\"added_tokens\"");
    if (added == std::string::npos) return;
    const size_t open = json.find('[', added);
    if (open == std::string::npos) return;
    size_t pos = open + 1;
    while (pos < json.size()) {
        const size_t b = json.find('{', pos);
        if (b == std::string::npos) break;
        size_t e = b + 1;
        bool in_str = false;
        while (e < json.size()) {
            if (json[e] == '"' && json[e - 1] != '\\') in_str = !in_str;
            else if (!in_str && json[e] == '}') break;
            e++;
        }
        if (e >= json.size()) break;
        const std::string obj = json.substr(b, e - b + 1);
        if (obj.find("\"special\"") != std::string::npos && obj.find("true") != std::string::npos) {
            const int id = json_int_after(obj, "id");
            size_t cs = obj.find("\"content\"");
            if (cs != std::string::npos && (cs = obj.find('"', cs + 9)) != std::string::npos) {
                const size_t ce = obj.find('"', cs + 1);
                if (ce != std::string::npos) {
                    const std::string content = obj.substr(cs + 1, ce - cs - 1);
                    if (id > 2 && content.size() > 1) tok->special_tokens.push_back({content, id});
                    if (content == "</s>" && id != tok->eos_id) tok->eos_id = id;
                }
            }
        }
        pos = e + 1;
        const size_t nxt = json.find_first_not_of(" \t\n\r,", pos);
        if (nxt != std::string::npos && json[nxt] == ']') break;
    }
    std::stable_sort(tok->special_tokens.begin(), tok->special_tokens.end(),
                     [](const SpecialToken& a, const SpecialToken& b) { return a.text.size() > b.text.size(); });
}

// engine/tokenizer.cpp:366-425: special-token texts are cut out of the input (first the longest that matches at the
// current offset), the stretches between them are encoded on their own
std::vector<int> encode_with_special(Tokenizer* tok, const std::string& text)
{
    if (tok->special_tokens.empty()) return encode_plain(tok, text);
    std::vector<int> ids;
    size_t pos = 0;
    while (pos < text.size()) {
        bool matched = false;
        for (const SpecialToken& st : tok->special_tokens)
            if (!st.text.empty() && text.compare(pos, st.text.size(), st.text) == 0) {
                ids.push_back(st.id);
                pos += st.text.size();
                matched = true;
                break;
            }
        if (matched) continue;
        size_t stop = text.size();
        for (const SpecialToken& st : tok->special_tokens) {
            if (st.text.empty()) continue;
            const size_t at = text.find(st.text, pos);
            if (at != std::string::npos && at < stop) stop = at;
        }
        const std::vector<int> seg = encode_plain(tok, text.substr(pos, stop - pos));
        ids.insert(ids.end(), seg.begin(), seg.end());
        pos = stop;
    }
    return ids;
}

}  // namespace

Tokenizer* load_tokenizer(const std::string& model_path)
{
    // sentencepiece model first, like the reference (engine/tokenizer.cpp:332-346)
    const std::string sp_path = model_path + "/tokenizer.model";
    if (std::ifstream(sp_path, std::ios::binary)) {
        auto* sp = new SpModel();
        const std::string err = sp->load(sp_path);
        if (err.empty()) {
            auto* tok = new Tokenizer();
            tok->sp_model = sp;
            tok->bos_id = sp->bos_id;
            tok->eos_id = sp->eos_id;
            tok->vocab_size = (int)sp->pieces.size();
            tok->type = 0;
            printf("  Tokenizer: sentencepiece, vocab=%d bos=%d eos=%d\n", tok->vocab_size, tok->bos_id, tok->eos_id);
            load_special_tokens(tok, model_path);
            return tok;
        }
        fprintf(stderr, "tokenizer: %s: %s\n", sp_path.c_str(), err.c_str());
        delete sp;
    }
    int bos = 0, eos = 0;
    BpeModel* m = load_bpe(model_path, &bos, &eos);
    if (!m) {
        fprintf(stderr, "No tokenizer found in %s (tried tokenizer.model, and vocab.bin + merges.bin)\n", model_path.c_str());
        return nullptr;
    }
    auto* tok = new Tokenizer();
    tok->sp_model = m;
    tok->bos_id = bos;
    tok->eos_id = eos;
    tok->vocab_size = (int)m->id_to_token.size();
    tok->type = 1;
    printf("  Tokenizer: HF BPE (binary), vocab=%d bos=%d eos=%d merges=%zu\n", tok->vocab_size, bos, eos, m->merges.size());
    return tok;
}

void free_tokenizer(Tokenizer* tok)
{
    if (!tok) return;
    if (tok->type == 0) delete (SpModel*)tok->sp_model;
    else delete (BpeModel*)tok->sp_model;
    delete tok;
}

std::vector<int> tokenize(Tokenizer* tok, const std::string& text)
{
    std::vector<int> ids = encode_with_special(tok, text);
    ids.insert(ids.begin(), tok->bos_id);
    return ids;
}

std::string detokenize(Tokenizer* tok, const std::vector<int>& tokens)
{
    if (tok->type == 0) return ((const SpModel*)tok->sp_model)->decode(tokens);
    const BpeModel* m = (const BpeModel*)tok->sp_model;
    std::string text;
    for (int id : tokens)
        if (id >= 0 && (size_t)id < m->id_to_token.size()) text += m->id_to_token[id];
    return text;
}

std::string detokenize_one(Tokenizer* tok, int token)
{
    for (const SpecialToken& st : tok->special_tokens)
        if (st.id == token) return st.text;
    if (tok->type == 0) {
        // engine/tokenizer.cpp:484-506: the piece with every escaped blank as a space and a <0xXX> piece as its byte
        const std::string& piece = ((const SpModel*)tok->sp_model)->id_to_piece(token);
        std::string out;
        size_t i = 0;
        while (i < piece.size()) {
            if (piece.compare(i, 3, "\xE2\x96\x81") == 0) {
                out += ' ';
                i += 3;
            } else if (piece[i] == '<' && i + 5 < piece.size() && piece[i + 1] == '0' && piece[i + 2] == 'x') {
                const size_t close = piece.find('>', i);
                if (close != std::string::npos) {
                    out += (char)strtol(piece.substr(i + 3, close - i - 3).c_str(), nullptr, 16);
                    i = close + 1;
                } else {
                    out += piece[i++];
                }
            } else {
                out += piece[i++];
            }
        }
        return out;
    }
    const BpeModel* m = (const BpeModel*)tok->sp_model;
    if (token < 0 || (size_t)token >= m->id_to_token.size()) return "";
    // engine/tokenizer.cpp:452-479: at every offset the longest (4..1 bytes) stretch that is a byte-encoder
    // character becomes its byte; anything else passes through
    const std::string& t = m->id_to_token[token];
    std::string out;
    size_t i = 0;
    while (i < t.size()) {
        bool found = false;
        for (size_t len = 4; len >= 1; len--) {
            if (i + len > t.size()) continue;
            auto it = m->byte_decoder.find(t.substr(i, len));
            if (it != m->byte_decoder.end()) {
                out += (char)it->second;
                i += len;
                found = true;
                break;
            }
        }
        if (!found) out += t[i++];
    }
    return out;
}

// ---- C face (ctypes / cgo / JNI callers) ----
extern "C" {

void* t12_tokenizer_load(const char* model_dir) { return load_tokenizer(model_dir ? model_dir : ""); }
void t12_tokenizer_free(void* tok) { free_tokenizer((Tokenizer*)tok); }

int t12_tokenizer_info(void* tok, int* bos_id, int* eos_id, int* vocab_size)
{
    auto* t = (Tokenizer*)tok;
    if (!t) return -1;
    if (bos_id) *bos_id = t->bos_id;
    if (eos_id) *eos_id = t->eos_id;
    if (vocab_size) *vocab_size = t->vocab_size;
    return 0;
}

int t12_tokenizer_type(void* tok) { return tok ? ((Tokenizer*)tok)->type : -1; }

// Number of special tokens; with index >= 0 also copies that token's text (at most cap bytes) and id.
int t12_tokenizer_special(void* tok, int index, char* text_out, size_t cap, int* id_out)
{
    auto* t = (Tokenizer*)tok;
    if (!t) return -1;
    if (index >= 0 && index < (int)t->special_tokens.size()) {
        const SpecialToken& st = t->special_tokens[index];
        if (text_out && cap) {
            const size_t n = std::min(cap - 1, st.text.size());
            memcpy(text_out, st.text.data(), n);
            text_out[n] = 0;
        }
        if (id_out) *id_out = st.id;
    }
    return (int)t->special_tokens.size();
}

// Appends to Tokenizer::special_tokens, keeping the list longest-first (stable), the order the reference
// sorts it into (engine/tokenizer.cpp:136-140).
int t12_tokenizer_add_special(void* tok, const char* text, int id)
{
    auto* t = (Tokenizer*)tok;
    if (!t || !text || !*text) return -1;
    t->special_tokens.push_back({text, id});
    std::stable_sort(t->special_tokens.begin(), t->special_tokens.end(),
                     [](const SpecialToken& a, const SpecialToken& b) { return a.text.size() > b.text.size(); });
    return 0;
}

// tokenize(): writes at most cap ids and returns how many the text has (call again with more room if > cap).
int t12_tokenizer_encode(void* tok, const char* text, size_t len, int* ids_out, int cap)
{
    if (!tok || (!text && len)) return -1;
    const std::vector<int> ids = tokenize((Tokenizer*)tok, std::string(text ? text : "", len));
    for (size_t i = 0; i < ids.size() && (int)i < cap; i++) ids_out[i] = ids[i];
    return (int)ids.size();
}

static int copy_out(const std::string& s, char* out, size_t cap)
{
    if (out && cap) memcpy(out, s.data(), std::min(cap, s.size()));
    return (int)s.size();
}

// detokenize() / detokenize_one(): write at most cap bytes (no terminator), return the full length.
int t12_tokenizer_decode(void* tok, const int* ids, int n, char* out, size_t cap)
{
    if (!tok || (!ids && n)) return -1;
    return copy_out(detokenize((Tokenizer*)tok, std::vector<int>(ids, ids + n)), out, cap);
}

int t12_tokenizer_decode_one(void* tok, int id, char* out, size_t cap)
{
    if (!tok) return -1;
    return copy_out(detokenize_one((Tokenizer*)tok, id), out, cap);
}

}  // extern "C"
