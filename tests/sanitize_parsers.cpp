// Driver for the address/undefined-behaviour sanitizer build of the library's host-side file parsers
// (tokenizer.cpp, sp_model.cpp, and check_model_dir of model.cpp).  tests/test_host_sanitizers.py builds it with
// -fsanitize=address,undefined and feeds it well-formed, truncated and corrupted files; the parsers may refuse a
// file, they may not read or write out of bounds.  A finding ends the process with a non-zero status.
//
//   sanitize_parsers tok <text file> <dir>...     load_tokenizer, tokenize / detokenize the text, free
//   sanitize_parsers dir <dir>...                 check_model_dir
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iterator>
#include <string>
#include <vector>

#include "turbo/tokenizer.h"
#ifdef WITH_MODEL_DIR
#include "turbo/model.h"
#endif

int main(int argc, char** argv)
{
    if (argc < 3) return 2;
    if (!strcmp(argv[1], "tok")) {
        std::ifstream f(argv[2], std::ios::binary);
        const std::string text((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
        size_t loaded = 0, ids_total = 0;
        for (int i = 3; i < argc; i++) {
            Tokenizer* t = load_tokenizer(argv[i]);
            if (!t) continue;
            loaded++;
            std::vector<int> ids = tokenize(t, text);
            ids_total += ids.size();
            ids.push_back(-1);
            ids.push_back(t->vocab_size);
            ids.push_back(1 << 30);
            const std::string back = detokenize(t, ids);
            size_t shown = back.size();
            for (int id : ids) shown += detokenize_one(t, id).size();
            for (int id = 0; id < t->vocab_size; id++) shown += detokenize_one(t, id).size();
            if (shown == (size_t)-1) printf("?");
            free_tokenizer(t);
        }
        printf("tok: %zu of %d directories loaded, %zu ids\n", loaded, argc - 3, ids_total);
        return 0;
    }
#ifdef WITH_MODEL_DIR
    if (!strcmp(argv[1], "dir")) {
        int good = 0;
        for (int i = 2; i < argc; i++) {
            std::string err;
            if (check_model_dir(argv[i], err)) good++;
        }
        printf("dir: %d of %d directories consistent\n", good, argc - 2);
        return 0;
    }
#endif
    return 2;
}
