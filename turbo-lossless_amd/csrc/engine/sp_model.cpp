// sentencepiece BPE models without the sentencepiece library (see sp_model.h).  Host code only.
//
// File format: a serialized protocol buffer (sentencepiece_model.proto of the sentencepiece project):
//   ModelProto      1: repeated SentencePiece pieces, 2: TrainerSpec, 3: NormalizerSpec
//   SentencePiece   1: piece (string), 2: score (float), 3: type (enum, default NORMAL)
//   TrainerSpec     3: model_type (1 unigram, 2 BPE, ...), 24: treat_whitespace_as_suffix, 35: byte_fallback,
//                   40: unk_id, 44: unk_surface, 46: bos_piece, 47: eos_piece
//   NormalizerSpec  2: precompiled_charsmap, 3: add_dummy_prefix, 4: remove_extra_whitespaces, 5: escape_whitespaces
// Encoding is the library's published BPE procedure: normalise, split into UTF-8 characters (user-defined pieces
// stay whole), then repeatedly join the adjacent pair whose concatenation is the vocabulary piece with the highest
// score (leftmost on ties) until no pair is a piece; a symbol that is not a piece becomes <unk>, or its bytes'
// <0xXX> pieces when the model has byte fallback.
#include "sp_model.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iterator>
#include <queue>

namespace {

const char kSpace[] = "\xE2\x96\x81";       // U+2581, the escaped blank

struct Reader {
    const uint8_t* p;
    const uint8_t* end;
    bool ok = true;
    uint64_t varint()
    {
        uint64_t v = 0;
        for (int shift = 0; shift < 64 && p < end; shift += 7) {
            const uint8_t b = *p++;
            v |= (uint64_t)(b & 0x7F) << shift;
            if (!(b & 0x80)) return v;
        }
        ok = false;
        return 0;
    }
    Reader sub()
    {
        const uint64_t n = varint();
        if (!ok || n > (uint64_t)(end - p)) {
            ok = false;
            return Reader{p, p};
        }
        Reader r{p, p + n};
        p += n;
        return r;
    }
    void skip(int wire)
    {
        if (wire == 0) (void)varint();
        else if (wire == 1) p += 8;
        else if (wire == 2) (void)sub();
        else if (wire == 5) p += 4;
        else ok = false;
        if (p > end) ok = false;
    }
    std::string str() const { return std::string((const char*)p, (size_t)(end - p)); }
};

// one UTF-8 character at s[i]: its length, 1 for a byte that starts no valid sequence
int char_len(const std::string& s, size_t i, bool* valid)
{
    const uint8_t c = (uint8_t)s[i];
    int n = c < 0x80 ? 1 : (c >> 5) == 0x6 ? 2 : (c >> 4) == 0xE ? 3 : (c >> 3) == 0x1E ? 4 : 0;
    *valid = false;
    if (n == 0 || i + n > s.size()) return 1;
    uint32_t cp = n == 1 ? c : c & (0xFF >> (n + 1));
    for (int k = 1; k < n; k++) {
        const uint8_t d = (uint8_t)s[i + k];
        if ((d & 0xC0) != 0x80) return 1;
        cp = (cp << 6) | (d & 0x3F);
    }
    static const uint32_t lowest[5] = {0, 0, 0x80, 0x800, 0x10000};
    if (cp < lowest[n] || cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return 1;     // overlong, out of range, surrogate
    *valid = true;
    return n;
}

}  // namespace

std::string SpModel::load(const std::string& path)
{
    std::ifstream f(path, std::ios::binary);
    if (!f) return "cannot open";
    const std::vector<uint8_t> buf((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    Reader r{buf.data(), buf.data() + buf.size()};
    int model_type = 1;
    bool suffix_ws = false, has_charsmap = false;
    std::string bos_piece = "<s>", eos_piece = "</s>";
    while (r.ok && r.p < r.end) {
        const uint64_t key = r.varint();
        const int field = (int)(key >> 3), wire = (int)(key & 7);
        if (field == 1 && wire == 2) {
            Reader m = r.sub();
            Piece pc{"", 0.0f, NORMAL};
            while (m.ok && m.p < m.end) {
                const uint64_t k = m.varint();
                const int fd = (int)(k >> 3), w = (int)(k & 7);
                if (fd == 1 && w == 2) pc.text = m.sub().str();
                else if (fd == 2 && w == 5 && m.end - m.p >= 4) {
                    memcpy(&pc.score, m.p, 4);
                    m.p += 4;
                } else if (fd == 3 && w == 0) pc.type = (int)m.varint();
                else m.skip(w);
            }
            if (!m.ok) return "malformed piece";
            pieces.push_back(pc);
        } else if (field == 2 && wire == 2) {
            Reader m = r.sub();
            while (m.ok && m.p < m.end) {
                const uint64_t k = m.varint();
                const int fd = (int)(k >> 3), w = (int)(k & 7);
                if (w == 0) {
                    const uint64_t v = m.varint();
                    if (fd == 3) model_type = (int)v;
                    else if (fd == 24) suffix_ws = v != 0;
                    else if (fd == 35) byte_fallback = v != 0;
                    else if (fd == 40) unk_id = (int)v;
                } else if (w == 2 && (fd == 44 || fd == 46 || fd == 47)) {
                    const std::string sv = m.sub().str();
                    if (fd == 44) unk_surface = sv;
                    else if (fd == 46) bos_piece = sv;
                    else eos_piece = sv;
                } else m.skip(w);
            }
            if (!m.ok) return "malformed trainer_spec";
        } else if (field == 3 && wire == 2) {
            Reader m = r.sub();
            while (m.ok && m.p < m.end) {
                const uint64_t k = m.varint();
                const int fd = (int)(k >> 3), w = (int)(k & 7);
                if (w == 0) {
                    const uint64_t v = m.varint();
                    if (fd == 3) add_dummy_prefix = v != 0;
                    else if (fd == 4) remove_extra_whitespaces = v != 0;
                    else if (fd == 5) escape_whitespaces = v != 0;
                } else if (w == 2 && fd == 2) {
                    const Reader map = m.sub();
                    if (map.end > map.p) has_charsmap = true;
                }
                else m.skip(w);
            }
            if (!m.ok) return "malformed normalizer_spec";
        } else {
            r.skip(wire);
        }
    }
    if (!r.ok) return "not a sentencepiece model (protocol buffer does not parse)";
    if (pieces.empty()) return "no pieces";
    if (model_type != 2) return "model_type is not BPE (unigram / word / char models are not read by this build)";
    if (has_charsmap) return "the model normalises with a character map (only identity normalisation is built)";
    if (suffix_ws) return "treat_whitespace_as_suffix is not built";
    for (int b = 0; b < 256; b++) byte_id[b] = -1;
    for (int i = 0; i < (int)pieces.size(); i++) {
        const Piece& pc = pieces[i];
        if (pc.type == UNUSED) return "the model marks pieces unused (their resegmentation is not built)";
        if (pc.type == NORMAL || pc.type == USER_DEFINED) merge_ids.emplace(pc.text, i);
        else reserved_ids.emplace(pc.text, i);
        if (pc.type == USER_DEFINED && !pc.text.empty()) user_defined.push_back(pc.text);
        if (pc.type == BYTE && pc.text.size() == 6) byte_id[strtol(pc.text.c_str() + 3, nullptr, 16) & 255] = i;
    }
    std::stable_sort(user_defined.begin(), user_defined.end(),
                     [](const std::string& a, const std::string& b) { return a.size() > b.size(); });
    if (unk_id < 0 || unk_id >= (int)pieces.size() || pieces[unk_id].type != UNKNOWN) return "unk_id does not name the unknown piece";
    auto control = [&](const std::string& name) {
        auto it = reserved_ids.find(name);
        return it != reserved_ids.end() && pieces[it->second].type == CONTROL ? it->second : -1;
    };
    bos_id = control(bos_piece);
    eos_id = control(eos_piece);
    if (byte_fallback)
        for (int b = 0; b < 256; b++)
            if (byte_id[b] < 0) return "byte_fallback without all 256 byte pieces";
    return "";
}

const std::string& SpModel::id_to_piece(int id) const
{
    static const std::string none;
    return id >= 0 && id < (int)pieces.size() ? pieces[id].text : none;
}

int SpModel::piece_to_id(const std::string& piece) const
{
    auto it = reserved_ids.find(piece);
    if (it != reserved_ids.end()) return it->second;
    it = merge_ids.find(piece);
    return it != merge_ids.end() ? it->second : unk_id;
}

// The library's Normalizer::Normalize for the identity rule: one character at a time (a byte that is not UTF-8
// becomes U+FFFD), blanks escaped, and -- with remove_extra_whitespaces -- leading, trailing and repeated blanks
// dropped; a blank in front when add_dummy_prefix.
std::string SpModel::normalize(const std::string& text) const
{
    size_t i = 0;
    if (remove_extra_whitespaces)
        while (i < text.size() && text[i] == ' ') i++;
    std::string out;
    if (i >= text.size()) return out;
    const std::string blank = escape_whitespaces ? kSpace : " ";
    if (add_dummy_prefix) out += blank;
    bool prev_space = remove_extra_whitespaces;
    while (i < text.size()) {
        bool valid;
        const int n = char_len(text, i, &valid);
        if (!valid) {
            out += "\xEF\xBF\xBD";
            prev_space = false;
        } else if (text[i] == ' ') {
            if (!prev_space) out += blank;
            prev_space = remove_extra_whitespaces;
        } else {
            out.append(text, i, (size_t)n);
            prev_space = false;
        }
        i += (size_t)n;
    }
    if (remove_extra_whitespaces)
        while (out.size() >= blank.size() && out.compare(out.size() - blank.size(), blank.size(), blank) == 0)
            out.resize(out.size() - blank.size());
    return out;
}

std::vector<int> SpModel::encode(const std::string& text) const
{
    const std::string norm = normalize(text);
    struct Symbol {
        size_t begin, len;     // piece = norm[begin, begin + len); len 0 = merged away
        int prev, next;
        bool frozen;           // user-defined piece: takes no part in merging
    };
    std::vector<Symbol> sym;
    for (size_t i = 0; i < norm.size();) {
        size_t n = 0;
        bool frozen = false;
        for (const std::string& u : user_defined)
            if (norm.compare(i, u.size(), u) == 0) {
                n = u.size();
                frozen = true;
                break;
            }
        if (!n) {
            bool valid;
            n = (size_t)char_len(norm, i, &valid);
        }
        sym.push_back({i, n, (int)sym.size() - 1, -1, frozen});
        i += n;
    }
    std::vector<int> ids;
    if (sym.empty()) return ids;
    for (size_t k = 0; k + 1 < sym.size(); k++) sym[k].next = (int)k + 1;

    struct Pair {
        int left, right;
        float score;
        size_t size;
    };
    auto lower = [](const Pair& a, const Pair& b) { return a.score < b.score || (a.score == b.score && a.left > b.left); };
    std::priority_queue<Pair, std::vector<Pair>, decltype(lower)> agenda(lower);
    auto offer = [&](int l, int r) {
        if (l < 0 || r < 0 || sym[l].frozen || sym[r].frozen) return;
        auto it = merge_ids.find(norm.substr(sym[l].begin, sym[l].len + sym[r].len));
        if (it == merge_ids.end()) return;
        agenda.push({l, r, pieces[it->second].score, sym[l].len + sym[r].len});
    };
    for (size_t k = 1; k < sym.size(); k++) offer((int)k - 1, (int)k);
    while (!agenda.empty()) {
        const Pair top = agenda.top();
        agenda.pop();
        Symbol& L = sym[top.left];
        Symbol& R = sym[top.right];
        if (L.len == 0 || R.len == 0 || L.len + R.len != top.size) continue;      // one of the two has changed since
        L.len += R.len;
        L.next = R.next;
        if (R.next >= 0) sym[R.next].prev = top.left;
        R.len = 0;
        offer(L.prev, top.left);
        offer(top.left, L.next);
    }
    bool prev_unk = false;
    for (int k = 0; k >= 0; k = sym[k].next) {
        const std::string piece = norm.substr(sym[k].begin, sym[k].len);
        const int id = piece_to_id(piece);
        const bool unk = id == unk_id;
        if (unk && byte_fallback) {
            for (unsigned char c : piece) ids.push_back(byte_id[c]);
        } else if (!(unk && prev_unk)) {       // a run of unknown symbols is one <unk>
            ids.push_back(id);
        }
        prev_unk = unk && !byte_fallback;
    }
    return ids;
}

std::string SpModel::decode(const std::vector<int>& ids) const
{
    std::string out, bytes;
    bool at_start = true;       // no text yet: only control pieces (and dropped blanks)
    auto flush_bytes = [&]() {
        for (size_t i = 0; i < bytes.size();) {
            bool valid;
            const int n = char_len(bytes, i, &valid);
            if (valid) out.append(bytes, i, (size_t)n);
            else out += "\xEF\xBF\xBD";
            i += (size_t)n;
        }
        bytes.clear();
    };
    for (int id : ids) {
        if (id < 0 || id >= (int)pieces.size()) continue;
        const Piece& pc = pieces[id];
        if (pc.type == BYTE) {
            bytes += (char)(strtol(pc.text.c_str() + 3, nullptr, 16) & 255);
            at_start = false;
            continue;
        }
        flush_bytes();
        if (pc.type == CONTROL) continue;
        if (pc.type == UNKNOWN) {
            out += unk_surface;
            at_start = false;
            continue;
        }
        // the blank the encoder put in front is dropped again: the first piece's leading blank, and with
        // remove_extra_whitespaces every piece that is nothing but that blank until text begins
        size_t from = 0;
        if (at_start && (add_dummy_prefix || remove_extra_whitespaces) && pc.text.compare(0, 3, kSpace) == 0) from = 3;
        at_start = at_start && remove_extra_whitespaces && from == 3 && pc.text.size() == 3;
        for (size_t i = from; i < pc.text.size();) {
            if (pc.text.compare(i, 3, kSpace) == 0) {
                out += ' ';
                i += 3;
            } else {
                out += pc.text[i++];
            }
        }
    }
    flush_bytes();
    return out;
}
