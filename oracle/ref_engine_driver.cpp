// Test infrastructure, not part of the product: a command-line driver over the REFERENCE's host engine
// (engine/model.cpp, engine/inference.cpp, engine/sampler.cpp, compiled where they lie with their own headers by
// oracle/Makefile, target ref_engine) linked with this build's library for the kernel launchers those files declare
// (inference.cpp:7-41, sampler.cpp:4-5).  What runs is the reference's loader (derived escape tables and all), its
// forward_b1 / forward_b4 / forward_b8 / chunked dispatch (inference.cpp:198-712), its generate (:716-748) and its
// sampler -- every kernel launch of which lands in libturbo12.so.
//
//   reference_engine_driver <model_dir> <batch> <max_tokens> <prompt id> [<prompt id> ...]
//
// prints "tokens: t0 t1 ..." (the greedy stream of sequence 0) and leaves with 0.  With REF_DRIVER_TIMED=1 in the
// environment the same generate() call runs a second time under a clock and "timed: <seconds> <forward calls>" follows
// (prompt positions + generated tokens: the reference prefills one token per forward).
#include <cstdio>
#include <chrono>
#include <cstdlib>
#include <string>
#include <vector>

#include "inference.h"
#include "model.h"
#include "sampler.h"

int main(int argc, char** argv)
{
    if (argc < 5) {
        fprintf(stderr, "usage: %s <model_dir> <batch> <max_tokens> <prompt id> [<prompt id> ...]\n", argv[0]);
        return 1;
    }
    const int batch = atoi(argv[2]), max_tokens = atoi(argv[3]);
    std::vector<int> prompt;
    for (int i = 4; i < argc; i++) prompt.push_back(atoi(argv[i]));
    Model* model = load_model(argv[1]);
    if (!model) {
        fprintf(stderr, "load_model failed\n");
        return 2;
    }
    InferenceState* state = create_inference_state(model, batch, model->max_seq_len);
    if (!state) {
        fprintf(stderr, "create_inference_state failed\n");
        return 3;
    }
    init_sampler(batch);
    const std::vector<int> out = generate(state, prompt, max_tokens);
    printf("tokens:");
    for (int t : out) printf(" %d", t);
    printf("\n");
    const char* timed = getenv("REF_DRIVER_TIMED");
    if (timed && timed[0] == '1') {
        const auto t0 = std::chrono::steady_clock::now();
        const std::vector<int> again = generate(state, prompt, max_tokens);
        const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        printf("timed: %.6f %zu\n", sec, prompt.size() + again.size());
    }
    fflush(stdout);
    free_inference_state(state);
    free_model(model);
    return 0;
}
