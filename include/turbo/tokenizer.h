// Text <-> token ids for the split-12 engine: the reference's engine/tokenizer.h API
// (Tokenizer, load_tokenizer, free_tokenizer, tokenize, detokenize, detokenize_one --
// engine/tokenizer.h:5-23) with both of its backends (engine/tokenizer.cpp:328-351 picks them in this order):
//
// type 0 -- <dir>/tokenizer.model, a sentencepiece model.  The reference hands it to the sentencepiece library
//   (engine/tokenizer.cpp:12-29); here the file (a serialized ModelProto) is read directly and encoded with the
//   library's published BPE procedure: BPE models with identity normalisation, byte fallback and user-defined
//   pieces (the Llama-2 / Mistral tokenizers).  A unigram model, or one that normalises with a character map,
//   is reported and skipped.  Special tokens come from <dir>/tokenizer.json like in the reference
//   (engine/tokenizer.cpp:85-152).
//
// type 1 -- byte-level BPE tables, files written by the reference's engine/extract_tokenizer.py:66-104 or by this
//   package's tokenizer_files.extract:
//     vocab.bin         int32 n_vocab, bos_id, eos_id; per token uint16 length + bytes (id = index)
//     merges.bin        int32 n_merges; per merge uint16 len_a, uint16 len_b, bytes_a, bytes_b (rank = index)
//     byte_encoder.bin  256 x (uint8 length + UTF-8 bytes): byte -> printable character (optional; identity when absent)
//   Encoding follows the reference rule exactly (engine/tokenizer.cpp:295-326): the whole text, without
//   pre-tokenisation, is mapped byte by byte through the byte encoder; then for every merge in rank order every
//   adjacent (left, right) occurrence is joined, left to right; a symbol that is not in the vocabulary becomes
//   id 0.  The implementation does that in O(n log n) (rank-ordered queue over a linked list) instead of one pass
//   over the text per merge, with identical output for every merge table, also ones that list a pair twice or a
//   merge before the merges that build its parts.
//
// Not built: the direct tokenizer.json parse (engine/tokenizer.cpp:195-293), whose byte table stays empty so that
// it cannot encode; run the extractor once instead.
#pragma once
#include <string>
#include <vector>

struct SpecialToken {
    std::string text;
    int id;
};

struct Tokenizer {
    void* sp_model;    // backend handle
    int bos_id, eos_id;
    int vocab_size;
    int type;          // 0 = sentencepiece model, 1 = byte-level BPE tables
    std::vector<SpecialToken> special_tokens;  // longest first; matched greedily before encoding (type 0: from
                                               // tokenizer.json; type 1: empty after load, as in the reference)
};

// nullptr (and a message on stderr) when the directory holds neither a readable tokenizer.model nor
// vocab.bin + merges.bin.
Tokenizer* load_tokenizer(const std::string& model_path);
void free_tokenizer(Tokenizer* tok);
// bos_id followed by the ids of `text` (engine/tokenizer.cpp:427-431).
std::vector<int> tokenize(Tokenizer* tok, const std::string& text);
// Type 0: the text of the ids as the sentencepiece library decodes them.  Type 1: the vocabulary strings of the
// ids joined, still in their byte-encoder spelling; unknown ids are skipped (engine/tokenizer.cpp:433-449).
std::string detokenize(Tokenizer* tok, const std::vector<int>& tokens);
// One id as display text: a special token's text, else the piece with escaped blanks as spaces and <0xXX> as the
// byte (type 0), or the vocabulary string mapped back to bytes (type 1) (engine/tokenizer.cpp:451-506); "" for an
// id outside the vocabulary.
std::string detokenize_one(Tokenizer* tok, int token);
