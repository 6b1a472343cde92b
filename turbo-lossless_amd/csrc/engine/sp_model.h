// Reader and encoder for sentencepiece BPE models (tokenizer.model), the format the reference's first tokenizer
// backend hands to the sentencepiece library (engine/tokenizer.cpp:12-29).  Host code only; no protobuf or
// sentencepiece dependency: the model file is a serialized ModelProto, read here field by field.
//
// Supported: model_type BPE, identity normalisation (no precompiled character map) with the three whitespace
// rules (add_dummy_prefix, remove_extra_whitespaces, escape_whitespaces), byte fallback, user-defined pieces.
// That covers the Llama-2 / Mistral tokenizers the reference targets.  A unigram model, a model with a character
// map, or one with pieces marked unused fails to load with a message.
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

struct SpModel {
    enum PieceType { NORMAL = 1, UNKNOWN = 2, CONTROL = 3, USER_DEFINED = 4, UNUSED = 5, BYTE = 6 };
    struct Piece {
        std::string text;
        float score;
        int type;
    };
    std::vector<Piece> pieces;
    std::unordered_map<std::string, int> merge_ids;      // NORMAL / USER_DEFINED pieces: what merging may produce
    std::unordered_map<std::string, int> reserved_ids;   // every other piece
    std::vector<std::string> user_defined;               // longest first
    int byte_id[256];
    int unk_id = 0, bos_id = -1, eos_id = -1;
    bool byte_fallback = false;
    bool add_dummy_prefix = true, remove_extra_whitespaces = true, escape_whitespaces = true;
    std::string unk_surface = " \xE2\x81\x87 ";

    // Empty string on success, else what is wrong with the file.
    std::string load(const std::string& path);
    std::string normalize(const std::string& text) const;
    std::vector<int> encode(const std::string& text) const;          // SentencePieceProcessor::Encode(text, &ids)
    std::string decode(const std::vector<int>& ids) const;           // SentencePieceProcessor::Decode(ids, &text)
    const std::string& id_to_piece(int id) const;                    // "" for an id outside the vocabulary
    int piece_to_id(const std::string& piece) const;                 // unk_id when absent
};
