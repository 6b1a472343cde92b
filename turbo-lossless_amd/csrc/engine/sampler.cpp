// Greedy sampler (engine/sampler.cpp:11-32): device argmax, one D2H copy and
// one stream synchronisation per step.  The result buffer is kept per (device, stream) -- the reference has one for
// the process -- so that states sampling on their own streams do not share it.
#include "turbo/sampler.h"
#include "turbo/model.h"

#include <cstdio>
#include <map>
#include <mutex>
#include <utility>

extern "C" void launch_argmax(const float* logits, int* result, int n, hipStream_t stream);
extern "C" void launch_argmax_batch(const float* logits, int* results, int n_vocab, int batch_size, hipStream_t stream);

namespace {

struct ResultBuf {
    int* ptr = nullptr;
    int size = 0;
};
std::mutex g_mu;
std::map<std::pair<int, hipStream_t>, ResultBuf> g_result;
int g_min_size = 1;                                    // init_sampler's hint

int* result_buffer(int batch, hipStream_t stream)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    std::lock_guard<std::mutex> lock(g_mu);
    ResultBuf& b = g_result[{dev, stream}];
    const int want = batch > g_min_size ? batch : g_min_size;
    if (b.size < batch) {
        if (b.ptr) (void)hipFree(b.ptr);               // waits for the device: nothing still writes the old buffer
        b.ptr = nullptr;
        b.size = 0;
        if (hipMalloc((void**)&b.ptr, (size_t)want * sizeof(int)) != hipSuccess)
            engine_fail("GPU error: sampler buffer allocation failed (%d ids)", want);
        b.size = want;
    }
    return b.ptr;
}

}  // namespace

// Called by t12_release_stream: the buffer of (current device, stream) goes with the stream.
extern "C" __attribute__((visibility("hidden"))) void t12_sampler_release_stream(hipStream_t stream)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_result.find({dev, stream});
    if (it == g_result.end()) return;
    if (it->second.ptr) (void)hipFree(it->second.ptr);
    g_result.erase(it);
}

// The reference allocates its one buffer here (engine/sampler.cpp:11-16); here the size is remembered and every
// stream's buffer is created with at least that many ids on first use.
void init_sampler(int max_batch)
{
    std::lock_guard<std::mutex> lock(g_mu);
    if (max_batch > g_min_size) g_min_size = max_batch;
}

int sample_greedy(const float* logits_gpu, int n_vocab, hipStream_t stream)
{
    int* d = result_buffer(1, stream);
    launch_argmax(logits_gpu, d, n_vocab, stream);
    int result = 0;
    if (hipMemcpyAsync(&result, d, sizeof(int), hipMemcpyDeviceToHost, stream) != hipSuccess ||
        hipStreamSynchronize(stream) != hipSuccess)
        engine_fail("GPU error (sample_greedy): %s", hipGetErrorString(hipGetLastError()));
    return result;
}

void sample_greedy_batch(const float* logits_gpu, int* tokens_out, int n_vocab, int batch_size, hipStream_t stream)
{
    int* d = result_buffer(batch_size, stream);
    launch_argmax_batch(logits_gpu, d, n_vocab, batch_size, stream);
    if (hipMemcpyAsync(tokens_out, d, (size_t)batch_size * sizeof(int), hipMemcpyDeviceToHost, stream) != hipSuccess ||
        hipStreamSynchronize(stream) != hipSuccess)
        engine_fail("GPU error (sample_greedy_batch): %s", hipGetErrorString(hipGetLastError()));
}
