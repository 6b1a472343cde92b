// Decode loop: the layer wiring of the reference's forward_b1 / forward_b8 /
// forward_batch_tiled (engine/inference.cpp:198-366, 459-533, 572-666) on the
// gfx950 kernels of this library:
//   * wq|wk|wv and gate|up are ONE launch each (segment tables), with the escape
//     corrections fused, instead of 3 + 1 and 1 + 1 launches;
//   * RoPE and the INT8 KV store are one launch;
//   * B = 1 uses the decode-GEMV, every B > 1 the decode+GEMM (all sequences
//     run; the reference silently runs sequence 0 only for B not in {1,4,8,8k}).
// Like the reference's batched modes, the B sequences share ONE KV-cache region
// (kv_stride = 0, inference.cpp:427-435): the B > 1 modes are meant for B
// identical streams in lock-step, which is what generate() feeds.
#include "turbo/inference.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>

#include "t12_abi.h"
#include "turbo/sampler.h"

extern "C" {
void launch_embed_lookup(const int16_t*, const int*, float*, int, int, int, hipStream_t);
void launch_argmax_batch(const float*, int*, int, int, hipStream_t);
void launch_rms_norm_bf16_batch(const float*, const float*, int16_t*, int, float, int, hipStream_t);
void launch_add_rms_norm_bf16_batch(float*, const float*, const float*, int16_t*, int, float, int, hipStream_t);
void launch_sum_add_rms_norm_bf16_batch(float*, const float*, int, size_t, int, const float*, const float*, int16_t*, int,
                                        float, int, hipStream_t);
void launch_silu_mul_bf16_batch(const float*, const float*, int16_t*, int, int, hipStream_t);
void launch_rope_store_kv_batch(float*, float*, const float*, int8_t*, int8_t*, float*, float*, const int*, int, int,
                                int, int, int, float, int, hipStream_t);
void launch_rope_store_kv(float*, float*, const float*, int8_t*, int8_t*, float*, float*, int, int, int, int, int,
                          float, hipStream_t);
void launch_attention_all_heads(const float*, const int8_t*, const int8_t*, const float*, const float*, int16_t*, int,
                                int, int, int, int, float, hipStream_t);
void launch_attention_all_heads_batch(const float*, const int8_t*, const int8_t*, const float*, const float*, int16_t*,
                                      const int*, int, int, int, int, float, int, int, hipStream_t);
void launch_rope_store_attention_partials(float*, float*, const float*, int8_t*, int8_t*, float*, float*, int16_t*,
                                          const int*, int, int, int, int, float, float, int, const float*, int, size_t,
                                          int, int, hipStream_t);
void launch_rope_scaling(float, float, float, float);
void launch_rope_store_attention(float*, float*, const float*, int8_t*, int8_t*, float*, float*, int16_t*, const int*,
                                 int, int, int, int, float, float, int, int, hipStream_t);
void launch_rope_store_attention_regions(float*, float*, const float*, int8_t*, int8_t*, float*, float*, int16_t*,
                                         const int*, int, int, int, int, float, float, int, int, int, hipStream_t);
void t12_rope_store_attention_copies(float*, float*, const float*, int8_t*, int8_t*, float*, float*, int16_t*, const int*,
                                     int, int, int, int, float, float, int, int, hipStream_t);
void launch_rope_store_attention_partials_regions(float*, float*, const float*, int8_t*, int8_t*, float*, float*, int16_t*,
                                                  const int*, int, int, int, int, float, float, int, const float*, int,
                                                  size_t, int, int, int, hipStream_t);
}

namespace {

struct LayerSegs {
    T12Segment qkv[3], o[1], gateup[2], down[1];
};
struct Impl {
    std::vector<LayerSegs> layers;
    T12Segment head[1];
    bool fused_b1 = false;     // B = 1 takes the 5-launch-per-layer path
    bool checked = false;
    // pipelined greedy decoding: sampled tokens land in pinned host memory, two slots in rotation
    int* h_tokens[2] = {nullptr, nullptr};
    hipEvent_t sampled[2] = {nullptr, nullptr};
    // per-sequence KV caches owned by the state (create_inference_state_per_sequence):
    // int8 [n_layer][batch][max_seq][kv_dim] twice, scales fp32 [n_layer][batch][max_seq][n_head_kv] twice
    bool per_seq = false;
    int seq_len = 0;
    int8_t* pk = nullptr;
    int8_t* pv = nullptr;
    float* psk = nullptr;
    float* psv = nullptr;
    // prefill_rows: a state of that many rows on the same model, whose buffers carry a batch-1 state's prompt passes
    InferenceState* helper = nullptr;
    // pipelined decoding: the second logits buffer (the forward enqueued ahead of the host's look at a token writes
    // there, so the logits that produced an end-of-stream token are still in place when the loop stops)
    float* logits_alt = nullptr;
    // read once, when the state is created
    bool no_pipeline = false;
};

// Where a forward reads and writes the KV cache: layer l of sequence b starts at
// k + l * layer_kv + b * kv_stride (scales: sk + l * layer_sc + b * kv_stride / head_dim).
struct KvView {
    int8_t* k;
    int8_t* v;
    float* sk;
    float* sv;
    size_t layer_kv, layer_sc;
    int kv_stride;      // 0: every row of the batch works on one region
    int max_seq;
    // 0: a region is [position][kv head][head_dim], the reference's layout (engine/model.h:58-63) -- the model's own
    // cache.  > 0: [kv head][head_major positions][head_dim], scales [kv head][head_major] -- the per-sequence caches,
    // which only this engine reads: a (sequence, KV head) workgroup of the attention kernel then streams contiguous memory.
    int head_major;
};

// RoPE + KV store + attention on either layout
void rope_store_attention(const KvView& kv, float* q, float* k, const float* v, int8_t* ck, int8_t* cv, float* sk, float* sv,
                          int16_t* out, const int* positions, int position, int n_head, int n_head_kv, int head_dim,
                          float theta, float scale, int B, hipStream_t st, bool copies = false)
{
    if (copies && kv.kv_stride == 0)
        t12_rope_store_attention_copies(q, k, v, ck, cv, sk, sv, out, positions, position, n_head, n_head_kv, head_dim, theta,
                                        scale, B, kv.head_major, st);
    else if (kv.head_major)
        launch_rope_store_attention_regions(q, k, v, ck, cv, sk, sv, out, positions, position, n_head, n_head_kv, head_dim,
                                            theta, scale, B, kv.kv_stride, kv.head_major, st);
    else
        launch_rope_store_attention(q, k, v, ck, cv, sk, sv, out, positions, position, n_head, n_head_kv, head_dim, theta,
                                    scale, B, kv.kv_stride, st);
}

enum LogitsMode { LOGITS_ALL, LOGITS_LAST_ROW, LOGITS_NONE };

void check_gpu(hipError_t e, const char* what)
{
    if (e != hipSuccess) {
        engine_fail("GPU error (%s): %s", what, hipGetErrorString(e));
    }
}

T12Segment seg_of(const CompressedWeight& w, float* out, int out_stride)
{
    if (!w.split_sm) {   // where the reference ends the process (inference.cpp:73,223,306)
        engine_fail("split12 data missing for weight %dx%d", w.M, w.K);
    }
    T12Segment s;
    s.sm = w.split_sm;
    s.gr = w.split_gr;
    const bool has = w.num_patches > 0 && w.row_offsets;
    s.row_off = has ? w.row_offsets : nullptr;
    s.cols = has ? w.patch_cols : nullptr;
    s.correct = has ? w.patch_correct : nullptr;
    s.wrong = has ? w.patch_wrong : nullptr;
    s.out = out;
    s.M = w.M;
    s.base_exp = w.base_exp;
    s.out_stride = out_stride;
    s.reserved = 0;
    return s;
}

void run_linear(const T12Segment* segs, int nseg, const int16_t* act, int K, int B, hipStream_t st)
{
    int rc;
    if (B == 1) rc = t12_gemv(segs, nseg, act, K, st);
    else rc = t12_gemm(segs, nseg, act, K, segs[0].out_stride, K, B, st);
    if (rc != T12_OK) {
        engine_fail("split-12 linear launch failed: %s", t12_last_error());
    }
}

// out = W . act, then x = out + residual (stored in out) and y = bf16(RMSNorm(x) * norm_w): the K-split
// partial sums of the GEMM are added up by the norm kernel itself (one launch less per linear).
void run_linear_add_norm(const T12Segment* seg, const int16_t* act, int K, int B, const float* residual,
                         const float* norm_w, float eps, int16_t* y, hipStream_t st)
{
    T12GemmPartials part;
    if (t12_gemm_deferred(seg, 1, act, K, seg->out_stride, K, B, &part, st) != T12_OK) {
        engine_fail("split-12 linear launch failed: %s", t12_last_error());
    }
    if (part.nsplit > 1)
        launch_sum_add_rms_norm_bf16_batch(seg->out, part.ws, part.nsplit, part.split_stride, part.ld, residual, norm_w,
                                           y, seg->M, eps, B, st);
    else
        launch_add_rms_norm_bf16_batch(seg->out, residual, norm_w, y, seg->M, eps, B, st);
}

}  // namespace

InferenceState* create_inference_state(Model* model, int batch_size, int max_seq_len)
{
    (void)max_seq_len;   // the cache belongs to the model (engine/model.cpp:271-282)
    auto* s = new InferenceState();
    s->model = model;
    s->batch_size = batch_size;
    s->positions = new int[batch_size]();
    const ModelConfig& c = model->config;
    const int n = c.n_embd, n_ff = c.n_ff, n_vocab = c.n_vocab;
    const int kv_dim = c.n_head_kv * (n / c.n_head);
    const size_t bs = (size_t)batch_size;
    auto fbuf = [&](size_t count) {
        float* p = nullptr;
        check_gpu(hipMalloc((void**)&p, count * sizeof(float)), "hipMalloc");
        return p;
    };
    s->hidden = fbuf(bs * n);
    s->hidden2 = fbuf(bs * n);
    s->attn_out = fbuf(bs * n);
    s->q_buf = fbuf(bs * n);
    s->k_buf = fbuf(bs * kv_dim);
    s->v_buf = fbuf(bs * kv_dim);
    s->ffn_gate = fbuf(bs * n_ff);
    s->ffn_up = fbuf(bs * n_ff);
    s->ffn_down = fbuf(bs * n);    // output of w_down on the fused B = 1 path
    s->logits = fbuf(bs * n_vocab);
    s->attn_scores_buf = nullptr;
    check_gpu(hipMalloc((void**)&s->d_positions, bs * sizeof(int)), "hipMalloc");
    check_gpu(hipMalloc((void**)&s->d_tokens, bs * sizeof(int)), "hipMalloc");
    const size_t max_act = (size_t)std::max(n, n_ff);
    check_gpu(hipMalloc((void**)&s->bf16_act, bs * max_act * sizeof(int16_t)), "hipMalloc");
    check_gpu(hipMalloc((void**)&s->bf16_act2, bs * max_act * sizeof(int16_t)), "hipMalloc");
    check_gpu(hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking), "stream");
    check_gpu(hipStreamCreateWithFlags(&s->stream2, hipStreamNonBlocking), "stream");
    check_gpu(hipEventCreateWithFlags(&s->sync_event, hipEventDisableTiming), "event");
    s->patch_descs_gpu = nullptr;

    auto* impl = new Impl();
    impl->layers.resize(c.n_layer);
    const char* nofuse = getenv("TURBO_NO_FUSE");     // debugging aid: one kernel per reference kernel
    impl->fused_b1 = !(nofuse && nofuse[0] == '1');   // confirmed against the tensors at the first forward
    impl->no_pipeline = getenv("TURBO_NO_PIPELINE") != nullptr;   // the reference's order: sample, wait, forward
    // the pipelined decode loop keeps the logits of the previous step while the next forward overwrites
    // state->logits: its second buffer belongs to the state's memory budget, not to the first decode call
    if (!impl->no_pipeline) impl->logits_alt = fbuf(bs * n_vocab);
    s->impl = impl;
    init_sampler(batch_size);
    return s;
}

// Extension (the reference shares one cache region across the batch, inference.cpp:427-435): a state whose
// sequences are independent -- own KV cache region each, own tokens, own positions.
InferenceState* create_inference_state_per_sequence(Model* model, int batch_size, int max_seq_len)
{
    const ModelConfig& c = model->config;
    const int head_dim = c.n_embd / c.n_head;
    const size_t kv_dim = (size_t)c.n_head_kv * head_dim;
    if (batch_size < 1 || max_seq_len < 1 || (size_t)max_seq_len * kv_dim > 0x7FFFFFFFu) {
        fprintf(stderr, "ERROR: per-sequence KV cache: batch %d x %d positions is not a usable shape\n", batch_size,
                max_seq_len);
        return nullptr;
    }
    const size_t rows = (size_t)c.n_layer * batch_size * max_seq_len;
    size_t free_b = 0, total_b = 0;
    (void)hipMemGetInfo(&free_b, &total_b);
    const size_t need = 2 * rows * kv_dim + 2 * rows * c.n_head_kv * sizeof(float);
    if (need > free_b) {
        fprintf(stderr, "ERROR: per-sequence KV cache needs %.1f GB, %.1f GB free\n", need / 1e9, free_b / 1e9);
        return nullptr;
    }
    InferenceState* s = create_inference_state(model, batch_size, max_seq_len);
    Impl* impl = (Impl*)s->impl;
    impl->per_seq = true;
    impl->seq_len = max_seq_len;
    check_gpu(hipMalloc((void**)&impl->pk, rows * kv_dim), "hipMalloc");
    check_gpu(hipMalloc((void**)&impl->pv, rows * kv_dim), "hipMalloc");
    check_gpu(hipMalloc((void**)&impl->psk, rows * c.n_head_kv * sizeof(float)), "hipMalloc");
    check_gpu(hipMalloc((void**)&impl->psv, rows * c.n_head_kv * sizeof(float)), "hipMalloc");
    printf("  Per-sequence KV cache: %d x %d positions, %.2f GB\n", batch_size, max_seq_len, need / 1e9);
    return s;
}

void free_inference_state(InferenceState* state)
{
    if (!state) return;
    delete[] state->positions;
    for (void* p : {(void*)state->hidden, (void*)state->hidden2, (void*)state->attn_out, (void*)state->q_buf,
                    (void*)state->k_buf, (void*)state->v_buf, (void*)state->ffn_gate, (void*)state->ffn_up,
                    (void*)state->ffn_down, (void*)state->logits, (void*)state->attn_scores_buf,
                    (void*)state->d_positions, (void*)state->d_tokens, (void*)state->bf16_act,
                    (void*)state->bf16_act2, state->patch_descs_gpu})
        if (p) (void)hipFree(p);
    if (state->stream) {
        (void)t12_release_stream(state->stream);          // the library's per-stream buffers go with the stream
        (void)hipStreamDestroy(state->stream);
    }
    if (state->stream2) {
        (void)t12_release_stream(state->stream2);
        (void)hipStreamDestroy(state->stream2);
    }
    if (state->sync_event) (void)hipEventDestroy(state->sync_event);
    Impl* impl = (Impl*)state->impl;
    if (impl) {
        for (int i = 0; i < 2; i++) {
            if (impl->h_tokens[i]) (void)hipHostFree(impl->h_tokens[i]);
            if (impl->sampled[i]) (void)hipEventDestroy(impl->sampled[i]);
        }
        for (void* p : {(void*)impl->pk, (void*)impl->pv, (void*)impl->psk, (void*)impl->psv, (void*)impl->logits_alt})
            if (p) (void)hipFree(p);
        free_inference_state(impl->helper);
    }
    delete impl;
    delete state;
}

namespace {

bool exp_ok(const CompressedWeight& w) { return w.split_sm && w.base_exp >= 0 && w.base_exp <= 240; }

// Every tensor can take the fast decode-GEMV with fused prologues / epilogues.
bool fused_b1_eligible(const Model* m)
{
    const ModelConfig& c = m->config;
    if (c.n_embd % 16 || c.n_embd > 8192 || c.n_ff % 16 || c.n_layer < 1) return false;
    if (!exp_ok(m->output_proj)) return false;
    for (const auto& L : m->layers)
        for (const CompressedWeight* w : {&L.wq, &L.wk, &L.wv, &L.wo, &L.w_gate, &L.w_up, &L.w_down})
            if (!exp_ok(*w)) return false;
    return true;
}

void must(int rc, const char* what)
{
    if (rc != T12_OK) {
        engine_fail("%s failed: %s", what, t12_last_error());
    }
}

// B = 1 decode step in 5 launches per layer:
//   RMSNorm + wq|wk|wv                          t12_gemv_norm
//   RoPE + INT8 KV store + GQA attention        launch_rope_store_attention
//   wo + residual add                           t12_gemv_add
//   RMSNorm + gate|up + SiLU*mul                t12_gemv_swiglu_norm
//   w_down + residual add                       t12_gemv_add
// The residual stream ping-pongs between hidden and hidden2 (a norm prologue reads one and
// workgroup 0 writes the sum into the other); the additions the reference does in
// add_rms_norm_bf16_batch (inference.cpp:301,341-346) happen in the prologue of the next linear.
void forward_b1_fused(InferenceState* state, const int* token_ids, const KvView& kv)
{
    Model* m = state->model;
    const ModelConfig& c = m->config;
    hipStream_t st = state->stream;
    const int n = c.n_embd, n_ff = c.n_ff, head_dim = n / c.n_head;
    const int kv_dim = c.n_head_kv * head_dim;
    const float scale = 1.0f / sqrtf((float)head_dim);
    Impl* impl = (Impl*)state->impl;
    const int pos = state->positions[0];

    if (token_ids) (void)hipMemcpyAsync(state->d_tokens, token_ids, sizeof(int), hipMemcpyHostToDevice, st);
    launch_embed_lookup(m->token_embd, state->d_tokens, state->hidden, n, 1, c.n_vocab, st);

    float* h = state->hidden;          // residual stream (always complete: wo / w_down add it in their store)
    float* h_alt = state->hidden2;
    int16_t* bf16_a = state->bf16_act;
    int16_t* bf16_b = state->bf16_act2;

    for (int layer = 0; layer < c.n_layer; layer++) {
        TransformerLayer& L = m->layers[layer];
        LayerSegs& S = impl->layers[layer];
        S.qkv[0] = seg_of(L.wq, state->q_buf, n);
        S.qkv[1] = seg_of(L.wk, state->k_buf, kv_dim);
        S.qkv[2] = seg_of(L.wv, state->v_buf, kv_dim);
        must(t12_gemv_norm(S.qkv, 3, h, nullptr, L.attn_norm, c.rms_norm_eps, nullptr, n, st), "qkv decode-GEMV");

        const size_t kv_off = (size_t)layer * kv.layer_kv;
        const size_t sc_off = (size_t)layer * kv.layer_sc;
        KvView one = kv;
        one.kv_stride = 0;
        rope_store_attention(one, state->q_buf, state->k_buf, state->v_buf, kv.k + kv_off, kv.v + kv_off, kv.sk + sc_off,
                             kv.sv + sc_off, bf16_a, nullptr, pos, c.n_head, c.n_head_kv, head_dim, c.rope_theta, scale, 1,
                             st);

        S.o[0] = seg_of(L.wo, h_alt, n);
        must(t12_gemv_add(S.o, bf16_a, n, h, st), "wo decode-GEMV");                  // h_alt = h + wo . attn
        std::swap(h, h_alt);

        S.gateup[0] = seg_of(L.w_gate, nullptr, n_ff);
        S.gateup[1] = seg_of(L.w_up, nullptr, n_ff);
        must(t12_gemv_swiglu_norm(&S.gateup[0], &S.gateup[1], h, nullptr, L.ffn_norm, c.rms_norm_eps, nullptr, n, bf16_b, st),
             "gate|up decode-GEMV");

        S.down[0] = seg_of(L.w_down, h_alt, n);
        must(t12_gemv_add(S.down, bf16_b, n_ff, h, st), "w_down decode-GEMV");         // h_alt = h + w_down . ffn
        std::swap(h, h_alt);
    }
    impl->head[0] = seg_of(m->output_proj, state->logits, c.n_vocab);
    if (c.n_vocab >= 32768) {
        // thousands of workgroups would each rebuild the normalised activations: one small kernel
        // does it once instead (measured: 7 + 114 us against 139 us for the 128256-row head)
        launch_rms_norm_bf16_batch(h, m->output_norm, bf16_a, n, c.rms_norm_eps, 1, st);
        must(t12_gemv(impl->head, 1, bf16_a, n, st), "lm_head decode-GEMV");
    } else {
        must(t12_gemv_norm(impl->head, 1, h, nullptr, m->output_norm, c.rms_norm_eps, nullptr, n, st),
             "lm_head decode-GEMV");
    }
    state->positions[0] = pos + 1;
}


// The KV cache a state works on: its own per-sequence regions, or the model's one region.
KvView kv_view(const InferenceState* state)
{
    const Model* m = state->model;
    const ModelConfig& c = m->config;
    const Impl* impl = (const Impl*)state->impl;
    const int kv_dim = c.n_head_kv * (c.n_embd / c.n_head);
    KvView kv;
    if (impl->per_seq) {
        const size_t S = (size_t)impl->seq_len, B = (size_t)state->batch_size;
        kv = KvView{impl->pk, impl->pv, impl->psk, impl->psv, B * S * kv_dim, B * S * c.n_head_kv, (int)(S * kv_dim),
                    impl->seq_len, impl->seq_len};
    } else {
        kv = KvView{m->kv_cache_k, m->kv_cache_v, m->kv_scale_k, m->kv_scale_v, (size_t)m->max_seq_len * kv_dim,
                    (size_t)m->max_seq_len * c.n_head_kv, 0, m->max_seq_len, 0};
    }
    return kv;
}

// One pass of the layer stack over R rows (R <= batch_size) whose token ids are in state->d_tokens and, for
// R > 1, whose positions are in state->d_positions; pos0 = position of the row when R == 1, else the largest
// position of the rows (a length hint for the attention launch).  Logits: for every row into
// state->logits (LOGITS_ALL), for the last row only into logits_last (LOGITS_LAST_ROW), or not at all.
// copies: the rows are copies of one sequence at one position on a shared cache (the lock-step batch of forward()).
void forward_rows(InferenceState* state, int R, const KvView& kv, int pos0, LogitsMode lm, float* logits_last,
                  bool copies = false)
{
    Model* m = state->model;
    const ModelConfig& c = m->config;
    hipStream_t st = state->stream;
    const int B = R;
    const int n = c.n_embd, n_ff = c.n_ff, head_dim = n / c.n_head;
    const int kv_dim = c.n_head_kv * head_dim;
    const float scale = 1.0f / sqrtf((float)head_dim);
    Impl* impl = (Impl*)state->impl;

    launch_embed_lookup(m->token_embd, state->d_tokens, state->hidden, n, B, c.n_vocab, st);

    float* cur = state->hidden;    // residual stream
    float* res = state->hidden2;
    int16_t* bf16_a = state->bf16_act;
    int16_t* bf16_b = state->bf16_act2;

    for (int layer = 0; layer < c.n_layer; layer++) {
        TransformerLayer& L = m->layers[layer];
        LayerSegs& S = impl->layers[layer];
        if (layer == 0) launch_rms_norm_bf16_batch(cur, L.attn_norm, bf16_a, n, c.rms_norm_eps, B, st);

        S.qkv[0] = seg_of(L.wq, state->q_buf, n);
        S.qkv[1] = seg_of(L.wk, state->k_buf, kv_dim);
        S.qkv[2] = seg_of(L.wv, state->v_buf, kv_dim);
        T12GemmPartials qkv_part = {nullptr, 1, 0, 0};
        if (B > 1) {
            // a K-split q | k | v projection leaves its partial sums to the RoPE / KV-store kernel
            if (t12_gemm_deferred(S.qkv, 3, bf16_a, n, n, n, B, &qkv_part, st) != T12_OK) {
                engine_fail("split-12 linear launch failed: %s", t12_last_error());
            }
        } else {
            run_linear(S.qkv, 3, bf16_a, n, B, st);
        }

        const size_t kv_off = (size_t)layer * kv.layer_kv;
        const size_t sc_off = (size_t)layer * kv.layer_sc;
        // RoPE (Q, K) + INT8 KV store + GQA attention
        if (qkv_part.nsplit > 1 && kv.head_major)
            launch_rope_store_attention_partials_regions(state->q_buf, state->k_buf, state->v_buf, kv.k + kv_off,
                                                         kv.v + kv_off, kv.sk + sc_off, kv.sv + sc_off, bf16_a,
                                                         state->d_positions, pos0, c.n_head, c.n_head_kv, head_dim,
                                                         c.rope_theta, scale, B, qkv_part.ws, qkv_part.nsplit,
                                                         qkv_part.split_stride, qkv_part.ld, kv.kv_stride, kv.head_major, st);
        else if (qkv_part.nsplit > 1)
            launch_rope_store_attention_partials(state->q_buf, state->k_buf, state->v_buf, kv.k + kv_off, kv.v + kv_off,
                                                 kv.sk + sc_off, kv.sv + sc_off, bf16_a, state->d_positions, pos0,
                                                 c.n_head, c.n_head_kv, head_dim, c.rope_theta, scale, B, qkv_part.ws,
                                                 qkv_part.nsplit, qkv_part.split_stride, qkv_part.ld, kv.kv_stride, st);
        else
            rope_store_attention(kv, state->q_buf, state->k_buf, state->v_buf, kv.k + kv_off, kv.v + kv_off, kv.sk + sc_off,
                                 kv.sv + sc_off, bf16_a, B == 1 ? nullptr : state->d_positions, pos0, c.n_head, c.n_head_kv,
                                 head_dim, c.rope_theta, scale, B, st, copies);

        S.o[0] = seg_of(L.wo, res, n);
        if (B > 1) {
            run_linear_add_norm(S.o, bf16_a, n, B, cur, L.ffn_norm, c.rms_norm_eps, bf16_a, st);
        } else {
            run_linear(S.o, 1, bf16_a, n, B, st);
            launch_add_rms_norm_bf16_batch(res, cur, L.ffn_norm, bf16_a, n, c.rms_norm_eps, B, st);
        }

        S.gateup[0] = seg_of(L.w_gate, state->ffn_gate, n_ff);
        S.gateup[1] = seg_of(L.w_up, state->ffn_up, n_ff);
        const bool fuse_swiglu = B == 1 && n % 16 == 0 && L.w_gate.base_exp >= 0 && L.w_gate.base_exp <= 240 &&
                                 L.w_up.base_exp >= 0 && L.w_up.base_exp <= 240;
        if (fuse_swiglu) {      // gate|up decode-GEMV with the SiLU*mul epilogue: one launch, no fp32 round trip
            if (t12_gemv_swiglu(&S.gateup[0], &S.gateup[1], bf16_a, n, bf16_b, st) != T12_OK) {
                engine_fail("fused gate|up launch failed: %s", t12_last_error());
            }
        } else {
            // gate|up decode+GEMM with the SiLU*mul in its epilogue where the shape has such a kernel
            const int rc = B > 1 ? t12_gemm_swiglu(&S.gateup[0], &S.gateup[1], bf16_a, n, n, B, bf16_b, n_ff, st) : 1;
            if (rc < 0) {
                engine_fail("fused gate|up launch failed: %s", t12_last_error());
            }
            if (rc == 1) {
                run_linear(S.gateup, 2, bf16_a, n, B, st);
                launch_silu_mul_bf16_batch(state->ffn_gate, state->ffn_up, bf16_b, n_ff, B, st);
            }
        }

        S.down[0] = seg_of(L.w_down, cur, n);
        const float* next_norm = layer + 1 < c.n_layer ? m->layers[layer + 1].attn_norm : m->output_norm;
        if (B > 1) {
            run_linear_add_norm(S.down, bf16_b, n_ff, B, res, next_norm, c.rms_norm_eps, bf16_a, st);
        } else {
            run_linear(S.down, 1, bf16_b, n_ff, B, st);
            launch_add_rms_norm_bf16_batch(cur, res, next_norm, bf16_a, n, c.rms_norm_eps, B, st);
        }
    }
    if (c.n_layer == 0) launch_rms_norm_bf16_batch(cur, m->output_norm, bf16_a, n, c.rms_norm_eps, B, st);

    if (lm == LOGITS_ALL) {
        impl->head[0] = seg_of(m->output_proj, state->logits, c.n_vocab);
        run_linear(impl->head, 1, bf16_a, n, B, st);
    } else if (lm == LOGITS_LAST_ROW) {
        impl->head[0] = seg_of(m->output_proj, logits_last, c.n_vocab);
        run_linear(impl->head, 1, bf16_a + (size_t)(B - 1) * n, n, 1, st);
    }
}

}  // namespace

void forward(InferenceState* state, const int* token_ids)
{
    Model* m = state->model;
    const ModelConfig& c = m->config;
    hipStream_t st = state->stream;
    const int B = state->batch_size;
    Impl* impl = (Impl*)state->impl;

    // the RoPE table is library state shared by every model of the process: name this model's rule
    launch_rope_scaling(c.rope_scaling[0], c.rope_scaling[1], c.rope_scaling[2], c.rope_scaling[3]);

    const KvView kv = kv_view(state);
    int max_pos = 0;
    for (int b = 0; b < B; b++) max_pos = std::max(max_pos, state->positions[b]);
    if (max_pos >= kv.max_seq) {
        engine_fail("position %d exceeds the KV cache (%d)", max_pos, kv.max_seq);
    }
    if (B == 1 && impl->fused_b1) {
        if (!impl->checked) {
            impl->checked = true;
            impl->fused_b1 = fused_b1_eligible(m);
        }
        if (impl->fused_b1) {
            forward_b1_fused(state, token_ids, kv);
            return;
        }
    }
    if (token_ids) (void)hipMemcpyAsync(state->d_tokens, token_ids, B * sizeof(int), hipMemcpyHostToDevice, st);
    if (B > 1) (void)hipMemcpyAsync(state->d_positions, state->positions, B * sizeof(int), hipMemcpyHostToDevice, st);
    // with a position array the scalar position is only the attention launch's length hint: the longest row
    // A batch on one shared cache whose rows stand at one position is the reference's batched mode: copies of one
    // sequence (inference.cpp:430-435; rows with unlike tokens would overwrite each other's cache slot there too).
    bool copies = B > 1 && !impl->per_seq;
    for (int b = 1; b < B && copies; b++) copies = state->positions[b] == state->positions[0];
    forward_rows(state, B, kv, B > 1 ? max_pos : state->positions[0], LOGITS_ALL, nullptr, copies);
    for (int b = 0; b < B; b++) state->positions[b]++;
}

// Batched prefill (extension; the reference prompts one token per forward, inference.cpp:721-724): the n
// prompt tokens of ONE sequence go through the layer stack as the rows of a batch, up to batch_size at a
// time, at consecutive positions on that sequence's cache region.  Every row's K / V is stored before any
// row attends, and row t attends to positions <= its own, so this is the causal prompt pass; the linears
// run on the decode+GEMM kernels.  Only the last token's logits are computed (row `seq` of state->logits).
// A state on the model's shared region (lock-step copies) advances every row and gets the logits in every row.
void prefill(InferenceState* state, int seq, const int* token_ids, int n_tokens)
{
    Model* m = state->model;
    const ModelConfig& c = m->config;
    hipStream_t st = state->stream;
    const int B = state->batch_size;
    Impl* impl = (Impl*)state->impl;
    if (seq < 0 || seq >= B || n_tokens < 0) {
        engine_fail("prefill: sequence %d outside the batch of %d, or negative length", seq, B);
    }
    if (n_tokens == 0) return;
    if (B == 1) {                                   // nothing to batch over: the decode path, token by token
        for (int i = 0; i < n_tokens; i++) forward(state, token_ids + i);
        return;
    }
    launch_rope_scaling(c.rope_scaling[0], c.rope_scaling[1], c.rope_scaling[2], c.rope_scaling[3]);
    KvView kv = kv_view(state);
    const int head_dim = c.n_embd / c.n_head;
    const int p0 = state->positions[seq];
    if (p0 + n_tokens > kv.max_seq) {
        engine_fail("position %d exceeds the KV cache (%d)", p0 + n_tokens - 1, kv.max_seq);
    }
    // the rows of a chunk share this sequence's region
    kv.k += (size_t)seq * kv.kv_stride;
    kv.v += (size_t)seq * kv.kv_stride;
    kv.sk += (size_t)seq * (kv.kv_stride / head_dim);
    kv.sv += (size_t)seq * (kv.kv_stride / head_dim);
    kv.kv_stride = 0;
    float* row_logits = state->logits + (size_t)(impl->per_seq ? seq : 0) * c.n_vocab;
    std::vector<int> pos(B);
    for (int done = 0; done < n_tokens;) {
        const int R = std::min(B, n_tokens - done);
        const bool last = done + R == n_tokens;
        for (int r = 0; r < R; r++) pos[r] = p0 + done + r;
        (void)hipMemcpyAsync(state->d_tokens, token_ids + done, R * sizeof(int), hipMemcpyHostToDevice, st);
        (void)hipMemcpyAsync(state->d_positions, pos.data(), R * sizeof(int), hipMemcpyHostToDevice, st);
        forward_rows(state, R, kv, p0 + done + (R > 1 ? R - 1 : 0), last ? LOGITS_LAST_ROW : LOGITS_NONE, row_logits);
        // pos[] is reused by the next chunk: the copies above read it when they are issued (pageable memory)
        done += R;
    }
    if (impl->per_seq) {
        state->positions[seq] = p0 + n_tokens;
    } else {
        for (int b = 1; b < B; b++)
            (void)hipMemcpyAsync(state->logits + (size_t)b * c.n_vocab, row_logits, (size_t)c.n_vocab * sizeof(float),
                                 hipMemcpyDeviceToDevice, st);
        for (int b = 0; b < B; b++) state->positions[b] = p0 + n_tokens;
    }
}

// A batch-1 state has no rows to batch a prompt over; a helper state of `rows` rows on the same model lends its
// buffers: the prompt goes through the decode+GEMM kernels `rows` tokens per pass into THIS state's cache region,
// and the last token's logits land in this state's logits.  The helper works on its own stream, ordered after what
// this state has enqueued and before what it enqueues next.
void prefill_rows(InferenceState* state, const int* token_ids, int n_tokens, int rows)
{
    if (state->batch_size != 1) {
        engine_fail("prefill_rows is for states of batch size 1 (got %d): use prefill", state->batch_size);
    }
    if (rows <= 1 || n_tokens <= 1) {
        prefill(state, 0, token_ids, n_tokens);
        return;
    }
    Impl* impl = (Impl*)state->impl;
    if (impl->helper && impl->helper->batch_size != rows) {
        check_gpu(hipStreamSynchronize(impl->helper->stream), "hipStreamSynchronize");
        free_inference_state(impl->helper);
        impl->helper = nullptr;
    }
    if (!impl->helper) impl->helper = create_inference_state(state->model, rows, 0);
    InferenceState* h = impl->helper;
    const ModelConfig& c = state->model->config;
    launch_rope_scaling(c.rope_scaling[0], c.rope_scaling[1], c.rope_scaling[2], c.rope_scaling[3]);
    KvView kv = kv_view(state);                    // this state's region (batch 1: sequence 0)
    kv.kv_stride = 0;
    const int p0 = state->positions[0];
    if (p0 + n_tokens > kv.max_seq) {
        engine_fail("position %d exceeds the KV cache (%d)", p0 + n_tokens - 1, kv.max_seq);
    }
    check_gpu(hipEventRecord(state->sync_event, state->stream), "hipEventRecord");
    check_gpu(hipStreamWaitEvent(h->stream, state->sync_event, 0), "hipStreamWaitEvent");
    std::vector<int> pos(rows);
    for (int done = 0; done < n_tokens;) {
        const int R = std::min(rows, n_tokens - done);
        const bool last = done + R == n_tokens;
        for (int r = 0; r < R; r++) pos[r] = p0 + done + r;
        (void)hipMemcpyAsync(h->d_tokens, token_ids + done, R * sizeof(int), hipMemcpyHostToDevice, h->stream);
        (void)hipMemcpyAsync(h->d_positions, pos.data(), R * sizeof(int), hipMemcpyHostToDevice, h->stream);
        forward_rows(h, R, kv, p0 + done + (R > 1 ? R - 1 : 0), last ? LOGITS_LAST_ROW : LOGITS_NONE, state->logits);
        done += R;
    }
    check_gpu(hipEventRecord(h->sync_event, h->stream), "hipEventRecord");
    check_gpu(hipStreamWaitEvent(state->stream, h->sync_event, 0), "hipStreamWaitEvent");
    state->positions[0] = p0 + n_tokens;
}

// Greedy decoding from the logits the state holds, `max_tokens` steps of (sample, forward).
// The reference's loop (inference.cpp:726-746) waits for every sampled token on the host before it
// enqueues the next forward, so the GPU idles for a host round trip per token.  Here the argmax
// writes the token ids straight into state->d_tokens and the next forward is enqueued on them at
// once (forward(state, nullptr)); the ids also travel to pinned host memory, and the host reads
// token t while the GPU already computes step t + 1.  Same tokens, same stop rule (id 2 of sequence
// 0 ends the stream when stop_on_eos): the one forward issued past an end-of-stream token is undone
// by stepping the positions back.  TURBO_NO_PIPELINE=1 restores the reference's order.
namespace {
// Sequence 0 sampling stop_a or stop_b (ids, -1 = none) ends the stream; on_token (may be empty) sees every id of
// sequence 0 that is kept, as soon as the host has it.
std::vector<int> decode_loop(InferenceState* state, int max_tokens, int stop_a, int stop_b, bool all_rows,
                             const std::function<void(int)>& on_token)
{
    std::vector<int> output;
    auto is_stop = [&](int t) { return (stop_a >= 0 && t == stop_a) || (stop_b >= 0 && t == stop_b); };
    const int n_vocab = state->model->config.n_vocab;
    const int bs = state->batch_size;
    hipStream_t st = state->stream;
    Impl* impl = (Impl*)state->impl;
    if (impl->no_pipeline) {
        std::vector<int> tokens(bs);
        for (int t = 0; t < max_tokens; t++) {
            if (bs == 1) tokens[0] = sample_greedy(state->logits, n_vocab, st);
            else sample_greedy_batch(state->logits, tokens.data(), n_vocab, bs, st);
            if (is_stop(tokens[0])) break;
            if (all_rows) output.insert(output.end(), tokens.begin(), tokens.end());
            else output.push_back(tokens[0]);
            if (on_token) on_token(tokens[0]);
            forward(state, tokens.data());
        }
        return output;
    }
    for (int i = 0; i < 2; i++) {
        if (!impl->h_tokens[i]) check_gpu(hipHostMalloc((void**)&impl->h_tokens[i], bs * sizeof(int)), "hipHostMalloc");
        if (!impl->sampled[i]) check_gpu(hipEventCreateWithFlags(&impl->sampled[i], hipEventDisableTiming), "hipEventCreate");
    }
    auto enqueue_sample = [&](int slot) {
        launch_argmax_batch(state->logits, state->d_tokens, n_vocab, bs, st);
        // ids -> pinned host memory by a kernel: a DMA-engine copy in the middle of the stream costs a
        // queue hand-over each way (~0.2 ms per token measured)
        must(t12_util_copy_i32(impl->h_tokens[slot], state->d_tokens, bs, st), "token copy");
        (void)hipEventRecord(impl->sampled[slot], st);
    };
    const int max_seq = kv_view(state).max_seq;
    if (max_tokens > 0) enqueue_sample(0);
    for (int t = 0; t < max_tokens; t++) {
        // The forward on token t is enqueued before the host has seen token t -- unless the cache is full: then the
        // host looks first, as the reference's order does, and a stop id ends the stream without an error.
        int max_pos = 0;
        for (int b = 0; b < bs; b++) max_pos = std::max(max_pos, state->positions[b]);
        const bool ahead = max_pos < max_seq;
        if (ahead) {
            std::swap(state->logits, impl->logits_alt);           // keep the logits token t came from
            forward(state, nullptr);                              // on the ids the argmax left in d_tokens
            if (t + 1 < max_tokens) enqueue_sample((t + 1) & 1);
        }
        check_gpu(hipEventSynchronize(impl->sampled[t & 1]), "hipEventSynchronize");
        const int tok = impl->h_tokens[t & 1][0];
        if (is_stop(tok)) {
            if (ahead) {
                for (int b = 0; b < bs; b++) state->positions[b]--;   // the forward on the end-of-stream id does not count
                std::swap(state->logits, impl->logits_alt);           // state->logits: those that produced the stop id
            }
            break;
        }
        if (all_rows) output.insert(output.end(), impl->h_tokens[t & 1], impl->h_tokens[t & 1] + bs);
        else output.push_back(tok);
        if (on_token) on_token(tok);
        if (!ahead) {
            forward(state, nullptr);                              // reports the full cache like the sequential order
            if (t + 1 < max_tokens) enqueue_sample((t + 1) & 1);
        }
    }
    check_gpu(hipStreamSynchronize(st), "hipStreamSynchronize");
    return output;
}
}  // namespace

std::vector<int> decode_greedy(InferenceState* state, int max_tokens, bool stop_on_eos)
{
    return decode_loop(state, max_tokens, stop_on_eos ? 2 : -1, -1, false, nullptr);
}

std::vector<int> decode_greedy_until(InferenceState* state, int max_tokens, int stop_id)
{
    return decode_loop(state, max_tokens, stop_id, -1, false, nullptr);
}

std::vector<int> decode_greedy_all(InferenceState* state, int max_tokens)
{
    return decode_loop(state, max_tokens, -1, -1, true, nullptr);
}

std::vector<int> generate(InferenceState* state, const std::vector<int>& prompt_tokens, int max_tokens)
{
    const int bs = state->batch_size;
    std::vector<int> tokens(bs);
    for (int i = 0; i < (int)prompt_tokens.size(); i++) {
        for (int s = 0; s < bs; s++) {
            state->positions[s] = i;
            tokens[s] = prompt_tokens[i];
        }
        forward(state, tokens.data());
    }
    return decode_greedy(state, max_tokens, true);
}

// engine/main.cpp:147-173: the cache rows [discard, current_pos) of every layer move to [0, current_pos - discard),
// keys as stored (rotated for their old positions), scales along.  The reference issues one copy per array
// whose source and destination overlap whenever more than `discard` rows are kept; here the rows move in
// pieces of at most `discard` rows, front to back on the state's stream, so no copy overlaps itself.
void shift_context(InferenceState* state, int seq, int current_pos, int discard)
{
    const KvView kv = kv_view(state);
    const ModelConfig& c = state->model->config;
    const int hd = c.n_embd / c.n_head, nkv = c.n_head_kv, kv_dim = nkv * hd;
    if (seq < 0 || seq >= state->batch_size || discard < 0 || discard > current_pos || current_pos > kv.max_seq) {
        engine_fail("shift_context(seq %d, current_pos %d, discard %d) outside the cache (%d sequences, %d positions)",
                seq, current_pos, discard, state->batch_size, kv.max_seq);
    }
    const int keep = current_pos - discard;
    if (discard == 0 || keep == 0) return;
    const size_t seq_kv = (size_t)seq * kv.kv_stride, seq_sc = seq_kv / hd;
    hipStream_t st = state->stream;
    for (int layer = 0; layer < c.n_layer; layer++) {
        int8_t* k = kv.k + layer * kv.layer_kv + seq_kv;
        int8_t* v = kv.v + layer * kv.layer_kv + seq_kv;
        float* sk = kv.sk + layer * kv.layer_sc + seq_sc;
        float* sv = kv.sv + layer * kv.layer_sc + seq_sc;
        for (int done = 0; done < keep; done += discard) {
            const size_t rows = (size_t)std::min(discard, keep - done);
            const size_t to = (size_t)done, from = (size_t)done + discard;
            if (kv.head_major) {                                  // every KV head's rows are a block of their own
                const size_t S = (size_t)kv.head_major;
                for (int h = 0; h < nkv; h++) {
                    check_gpu(hipMemcpyAsync(k + (h * S + to) * hd, k + (h * S + from) * hd, rows * hd, hipMemcpyDeviceToDevice, st), "shift K");
                    check_gpu(hipMemcpyAsync(v + (h * S + to) * hd, v + (h * S + from) * hd, rows * hd, hipMemcpyDeviceToDevice, st), "shift V");
                    check_gpu(hipMemcpyAsync(sk + h * S + to, sk + h * S + from, rows * sizeof(float), hipMemcpyDeviceToDevice, st),
                              "shift K scales");
                    check_gpu(hipMemcpyAsync(sv + h * S + to, sv + h * S + from, rows * sizeof(float), hipMemcpyDeviceToDevice, st),
                              "shift V scales");
                }
                continue;
            }
            check_gpu(hipMemcpyAsync(k + to * kv_dim, k + from * kv_dim, rows * kv_dim, hipMemcpyDeviceToDevice, st), "shift K");
            check_gpu(hipMemcpyAsync(v + to * kv_dim, v + from * kv_dim, rows * kv_dim, hipMemcpyDeviceToDevice, st), "shift V");
            check_gpu(hipMemcpyAsync(sk + to * nkv, sk + from * nkv, rows * nkv * sizeof(float), hipMemcpyDeviceToDevice, st),
                      "shift K scales");
            check_gpu(hipMemcpyAsync(sv + to * nkv, sv + from * nkv, rows * nkv * sizeof(float), hipMemcpyDeviceToDevice, st),
                      "shift V scales");
        }
    }
}

// One turn of the reference's interactive loop, engine/main.cpp:139-203, without its printing.
std::vector<int> chat_turn(InferenceState* state, int* current_pos, const std::vector<int>& turn_tokens, int max_tokens,
                           int bos_id, int eos_id, int* discarded, const std::function<void(int)>& on_token, int prompt_rows)
{
    if (discarded) *discarded = 0;
    if (state->batch_size != 1) {
        engine_fail("chat_turn needs a state of batch size 1 (got %d)", state->batch_size);
    }
    std::vector<int> tokens = turn_tokens;
    int pos = *current_pos;
    if (pos > 0 && !tokens.empty() && tokens[0] == bos_id) tokens.erase(tokens.begin());   // BOS only opens the first turn (:141-143)
    const int max_seq = kv_view(state).max_seq;
    const int shift_limit = 1024;                                                            // :148
    const int headroom = (int)tokens.size() + max_tokens + 64;
    if (pos + headroom > max_seq || pos > shift_limit) {
        const int discard = pos / 2;
        shift_context(state, 0, pos, discard);
        pos -= discard;
        if (discarded) *discarded = discard;
    }
    state->positions[0] = pos;
    // one forward per new token like the reference (:181-184), or prompt_rows tokens per pass
    prefill_rows(state, tokens.data(), (int)tokens.size(), prompt_rows);
    std::vector<int> out = decode_loop(state, max_tokens, eos_id, bos_id, false, on_token);   // :192-202
    const int eos_tok = eos_id > 0 ? eos_id : 2;                 // the turn's end enters the context (:207-213)
    forward(state, &eos_tok);
    *current_pos = state->positions[0];
    return out;
}
