// Greedy sampler (engine/sampler.cpp:11-32): device argmax, one D2H copy and
// one stream synchronisation per step.
#include "turbo/sampler.h"
#include "turbo/model.h"

#include <cstdio>
#include <cstdlib>

extern "C" void launch_argmax(const float* logits, int* result, int n, hipStream_t stream);
extern "C" void launch_argmax_batch(const float* logits, int* results, int n_vocab, int batch_size, hipStream_t stream);

static int* s_d_result = nullptr;
static int s_d_result_size = 0;

void init_sampler(int max_batch)
{
    if (max_batch <= s_d_result_size) return;
    if (s_d_result) (void)hipFree(s_d_result);
    if (hipMalloc((void**)&s_d_result, (size_t)max_batch * sizeof(int)) != hipSuccess) {
        engine_fail("GPU error: sampler buffer allocation failed");
    }
    s_d_result_size = max_batch;
}

int sample_greedy(const float* logits_gpu, int n_vocab, hipStream_t stream)
{
    if (!s_d_result) init_sampler(1);
    launch_argmax(logits_gpu, s_d_result, n_vocab, stream);
    int result = 0;
    (void)hipMemcpyAsync(&result, s_d_result, sizeof(int), hipMemcpyDeviceToHost, stream);
    (void)hipStreamSynchronize(stream);
    return result;
}

void sample_greedy_batch(const float* logits_gpu, int* tokens_out, int n_vocab, int batch_size, hipStream_t stream)
{
    if (batch_size > s_d_result_size) init_sampler(batch_size);
    launch_argmax_batch(logits_gpu, s_d_result, n_vocab, batch_size, stream);
    (void)hipMemcpyAsync(tokens_out, s_d_result, (size_t)batch_size * sizeof(int), hipMemcpyDeviceToHost, stream);
    (void)hipStreamSynchronize(stream);
}
