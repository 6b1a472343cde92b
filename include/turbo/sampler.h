// Greedy sampling: the reference's engine/sampler.h API (sampler.h:5-11).
#pragma once
#include <hip/hip_runtime.h>

void init_sampler(int max_batch = 1);
int sample_greedy(const float* logits_gpu, int n_vocab, hipStream_t stream);
void sample_greedy_batch(const float* logits_gpu, int* tokens_out, int n_vocab, int batch_size, hipStream_t stream);
