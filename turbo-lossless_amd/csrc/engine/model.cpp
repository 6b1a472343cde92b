// Model store: reads the directory layout the reference's converter writes
// (engine/convert_model.py:57-62,127-152) into HBM, as engine/model.cpp:32-328
// does, with the file sizes checked against .dims; plus a GPU-side synthetic
// model generator and a writer of the same layout.
#include "turbo/model.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sys/stat.h>

#include "t12_abi.h"

extern "C" int t12_synth_normal_bf16(void*, size_t, uint64_t, float, float, float, void*);
extern "C" int t12_fill_f32(void*, size_t, float, void*);

void engine_fail(const char* fmt, ...)
{
    char text[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(text, sizeof text, fmt, ap);
    va_end(ap);
    fprintf(stderr, "ERROR: %s\n", text);
    throw EngineError(text);
}

namespace {

bool read_file(const std::string& path, std::vector<uint8_t>& data, bool quiet = false)
{
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) {
        if (!quiet) fprintf(stderr, "Cannot open: %s\n", path.c_str());
        data.clear();
        return false;
    }
    const std::streamoff size = f.tellg();
    f.seekg(0);
    data.resize((size_t)size);
    if (size > 0) f.read((char*)data.data(), size);
    return (bool)f;
}

bool gpu_ok(hipError_t e, const char* what)
{
    if (e == hipSuccess) return true;
    fprintf(stderr, "GPU error (%s): %s\n", what, hipGetErrorString(e));
    return false;
}

// Device copy of a host array; an allocation failure throws EngineError where the
// reference's GPU_CHECK (gpu_compat.h:94-101) ends the process.
template <typename T>
T* upload(const void* host, size_t count)
{
    if (count == 0) return nullptr;
    T* d = nullptr;
    if (!gpu_ok(hipMalloc((void**)&d, count * sizeof(T)), "hipMalloc")) engine_fail("cannot allocate %zu bytes of device memory", count * sizeof(T));
    if (!gpu_ok(hipMemcpy(d, host, count * sizeof(T), hipMemcpyHostToDevice), "hipMemcpy")) engine_fail("copy of %zu bytes to the device failed", count * sizeof(T));
    return d;
}

template <typename T>
T* device_alloc(size_t count)
{
    T* d = nullptr;
    if (!gpu_ok(hipMalloc((void**)&d, std::max<size_t>(count, 1) * sizeof(T)), "hipMalloc"))
        engine_fail("cannot allocate %zu bytes of device memory", std::max<size_t>(count, 1) * sizeof(T));
    return d;
}

void clear_weight(CompressedWeight& w)
{
    memset(&w, 0, sizeof w);
}

// Derived escape tables, the layout of engine/model.cpp:86-160 with WG = 256:
// row_base[r] = escapes before row r; esc_vals ordered (row, col % 256, ascending col);
// list of rows that hold an escape.  escape_counts is never built (the kernels
// here read the CSR list).
void build_escape_tables(CompressedWeight& w, const int32_t* row_off, const int32_t* cols, const int16_t* correct)
{
    const int WG = 256;
    std::vector<int32_t> row_base(w.M), nonempty;
    std::vector<int16_t> vals(w.num_patches);
    std::vector<int32_t> bucket(WG + 1);
    for (int r = 0; r < w.M; r++) {
        const int beg = row_off[r], end = row_off[r + 1];
        row_base[r] = beg;
        if (end == beg) continue;
        nonempty.push_back(r);
        std::fill(bucket.begin(), bucket.end(), 0);
        for (int p = beg; p < end; p++) bucket[cols[p] % WG + 1]++;
        for (int t = 0; t < WG; t++) bucket[t + 1] += bucket[t];
        for (int p = beg; p < end; p++) vals[beg + bucket[cols[p] % WG]++] = correct[p];   // cols ascend in a row
    }
    w.escape_row_base = upload<int32_t>(row_base.data(), row_base.size());
    w.escape_vals = upload<int16_t>(vals.data(), vals.size());
    w.escape_counts = nullptr;
    w.num_nonempty_rows = (int)nonempty.size();
    w.patch_nonempty_rows = upload<int32_t>(nonempty.data(), nonempty.size());
}


// ---------------------------------------------------------------- directory check (host only)
long long file_size(const std::string& path)
{
    struct stat st;
    if (stat(path.c_str(), &st) != 0 || !S_ISREG(st.st_mode)) return -1;
    return (long long)st.st_size;
}

bool fail(std::string& err, const std::string& what)
{
    err = what;
    return false;
}

// One tensor: .dims against the shape its role implies, the seven file sizes against .dims, and the CSR list's
// own invariants (row_off[0] == 0, non-decreasing, row_off[M] == P; columns inside the row and ascending in it).
bool check_tensor(const std::string& dir, const std::string& prefix, int want_M, int want_K, std::string& err)
{
    const std::string base = dir + "/" + prefix;
    std::ifstream df(base + ".dims");
    if (!df) return fail(err, prefix + ".dims is missing");
    long long M = 0, K = 0, P = 0, be = 0;
    if (!(df >> M >> K >> P) || M <= 0 || K <= 0 || P < 0 || M > 0x7FFFFFFF || K > 0x7FFFFFFF || P > 0x7FFFFFFF)
        return fail(err, prefix + ".dims is malformed");
    if (!(df >> be)) be = 0;                       // 4th field optional (engine/model.cpp:38-42)
    if (M != want_M || K != want_K)
        return fail(err, prefix + ": dims " + std::to_string(M) + " x " + std::to_string(K) + " but config.bin implies " +
                             std::to_string(want_M) + " x " + std::to_string(want_K));
    if (be < -1 || be > 254) return fail(err, prefix + ": base_exp " + std::to_string(be) + " outside -1..254");
    const long long n = M * K;
    if (file_size(base + ".sm.bin") != n || file_size(base + ".gr.bin") != (n + 1) / 2)
        return fail(err, prefix + ": .sm.bin / .gr.bin missing or not the size of " + std::to_string(M) + " x " + std::to_string(K));
    if (P == 0) return true;                       // the three list files may be empty or absent (model.cpp:47-68)
    if (file_size(base + ".row_off.bin") != (M + 1) * 4 || file_size(base + ".patch_cols.bin") != P * 4 ||
        file_size(base + ".patch_correct.bin") != P * 2 || file_size(base + ".patch_wrong.bin") != P * 2)
        return fail(err, prefix + ": escape list files do not match num_patches " + std::to_string(P));
    std::vector<uint8_t> ro, pc;
    if (!read_file(base + ".row_off.bin", ro, true) || !read_file(base + ".patch_cols.bin", pc, true))
        return fail(err, prefix + ": escape list files unreadable");
    const int32_t* r = (const int32_t*)ro.data();
    const int32_t* c = (const int32_t*)pc.data();
    if (r[0] != 0) return fail(err, prefix + ": row_off[0] is not 0");
    if (r[M] != P) return fail(err, prefix + ": row_off[M] is not num_patches");
    for (long long i = 0; i < M; i++)
        if (r[i + 1] < r[i]) return fail(err, prefix + ": row_off is not monotone");
    for (long long i = 0; i < M; i++)
        for (int32_t q = r[i]; q < r[i + 1]; q++) {
            if (c[q] < 0 || c[q] >= K) return fail(err, prefix + ": escape column out of range");
            if (q > r[i] && c[q] <= c[q - 1]) return fail(err, prefix + ": escape columns of a row do not ascend");
        }
    return true;
}

bool read_config(const std::string& model_path, ModelConfig& c, std::string& err)
{
    std::vector<uint8_t> buf;
    if (!read_file(model_path + "/config.bin", buf, true) || buf.size() < 36)
        return fail(err, "No config.bin found in " + model_path);
    struct { int32_t v[7]; float theta, eps; } raw;
    static_assert(sizeof raw == 36, "config.bin is 36 bytes");
    memcpy(&raw, buf.data(), sizeof raw);
    c.n_vocab = raw.v[0]; c.n_embd = raw.v[1]; c.n_head = raw.v[2]; c.n_head_kv = raw.v[3];
    c.n_layer = raw.v[4]; c.n_ff = raw.v[5]; c.n_ctx = raw.v[6];
    c.rope_theta = raw.theta; c.rms_norm_eps = raw.eps;
    c.rope_scaling[0] = c.rope_scaling[1] = c.rope_scaling[2] = c.rope_scaling[3] = 0.0f;
    std::vector<uint8_t> rs;
    if (read_file(model_path + "/rope_scaling.bin", rs, true)) {
        if (rs.size() != 16) return fail(err, "rope_scaling.bin in " + model_path + " is not 4 floats");
        memcpy(c.rope_scaling, rs.data(), 16);
        if (!(c.rope_scaling[0] > 0.0f) || !(c.rope_scaling[2] > c.rope_scaling[1]) || !(c.rope_scaling[3] > 0.0f))
            return fail(err, "rope_scaling.bin in " + model_path + " holds impossible values");
    }
    if (c.n_vocab <= 0 || c.n_embd <= 0 || c.n_head <= 0 || c.n_head_kv <= 0 || c.n_layer < 0 || c.n_ff <= 0 ||
        c.n_embd % c.n_head || c.n_head % c.n_head_kv)
        return fail(err, "config.bin in " + model_path + " holds an impossible shape");
    return true;
}

const char* const kTensorNames[7] = {"wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"};

// (rows, columns) of layer tensor `which` (order of kTensorNames) for a configuration
void tensor_shape(const ModelConfig& c, int which, int& M, int& K)
{
    const int n = c.n_embd, kv = c.n_head_kv * (c.n_embd / c.n_head);
    switch (which) {
        case 1: case 2: M = kv; K = n; break;
        case 4: case 5: M = c.n_ff; K = n; break;
        case 6: M = n; K = c.n_ff; break;
        default: M = n; K = n; break;
    }
}

bool load_compressed(const std::string& dir, const std::string& prefix, CompressedWeight& w)
{
    clear_weight(w);
    const std::string base = dir + "/" + prefix;
    std::ifstream df(base + ".dims");
    if (!df) {
        fprintf(stderr, "Missing: %s.dims\n", base.c_str());
        return false;
    }
    int M = 0, K = 0, P = 0, be = 0;
    if (!(df >> M >> K >> P) || M <= 0 || K <= 0 || P < 0) {
        fprintf(stderr, "ERROR: malformed %s.dims\n", base.c_str());
        return false;
    }
    if (!(df >> be)) be = 0;                       // 4th field optional (engine/model.cpp:38-42)
    const size_t n = (size_t)M * K;

    std::vector<uint8_t> sm, gr, ro, pc, pv, pw;
    if (!read_file(base + ".sm.bin", sm, true) || !read_file(base + ".gr.bin", gr, true) || sm.empty() || gr.empty()) {
        fprintf(stderr, "ERROR: split12 files missing for %s (need .sm.bin + .gr.bin)\n", prefix.c_str());
        return false;
    }
    if (sm.size() != n || gr.size() != (n + 1) / 2) {
        fprintf(stderr, "ERROR: %s: plane sizes %zu/%zu do not match dims %d x %d\n", prefix.c_str(), sm.size(),
                gr.size(), M, K);
        return false;
    }
    read_file(base + ".row_off.bin", ro, true);
    read_file(base + ".patch_cols.bin", pc, true);
    read_file(base + ".patch_correct.bin", pv, true);
    read_file(base + ".patch_wrong.bin", pw, true);
    if (P > 0) {
        const bool sizes_ok = ro.size() == (size_t)(M + 1) * 4 && pc.size() == (size_t)P * 4 &&
                              pv.size() == (size_t)P * 2 && pw.size() == (size_t)P * 2;
        if (!sizes_ok || ((const int32_t*)ro.data())[M] != P || ((const int32_t*)ro.data())[0] != 0) {
            fprintf(stderr, "ERROR: %s: escape list files do not match num_patches %d\n", prefix.c_str(), P);
            return false;
        }
        const int32_t* h_ro = (const int32_t*)ro.data();
        const int32_t* h_pc = (const int32_t*)pc.data();
        for (int r = 0; r < M; r++)
            if (h_ro[r + 1] < h_ro[r]) { fprintf(stderr, "ERROR: %s: row_off not monotone\n", prefix.c_str()); return false; }
        for (int p = 0; p < P; p++)
            if (h_pc[p] < 0 || h_pc[p] >= K) { fprintf(stderr, "ERROR: %s: escape column out of range\n", prefix.c_str()); return false; }
    }
    w.M = M;
    w.K = K;
    w.num_patches = P;
    w.base_exp = be;
    w.split_sm = upload<uint8_t>(sm.data(), sm.size());
    w.split_gr = upload<uint8_t>(gr.data(), gr.size());
    if (P > 0) {
        w.row_offsets = upload<int32_t>(ro.data(), M + 1);
        w.patch_cols = upload<int32_t>(pc.data(), P);
        w.patch_correct = upload<int16_t>(pv.data(), P);
        w.patch_wrong = upload<int16_t>(pw.data(), P);
        build_escape_tables(w, (const int32_t*)ro.data(), (const int32_t*)pc.data(), (const int16_t*)pv.data());
    }
    return true;
}

void free_weight(CompressedWeight& w)
{
    void* ptrs[] = {w.row_offsets, w.patch_cols, w.patch_correct, w.patch_wrong, w.escape_row_base, w.escape_counts,
                    w.escape_vals, w.split_sm,   w.split_gr,      w.patch_nonempty_rows};
    for (void* p : ptrs)
        if (p) (void)hipFree(p);
    clear_weight(w);
}

void alloc_kv_cache(Model* m, int max_seq)
{
    const ModelConfig& c = m->config;
    const int head_dim = c.n_embd / c.n_head;
    m->max_seq_len = std::max(max_seq, 128);
    const size_t kv = (size_t)c.n_layer * m->max_seq_len * c.n_head_kv * head_dim;
    const size_t sc = (size_t)c.n_layer * m->max_seq_len * c.n_head_kv;
    m->kv_cache_k = device_alloc<int8_t>(kv);
    m->kv_cache_v = device_alloc<int8_t>(kv);
    m->kv_scale_k = device_alloc<float>(sc);
    m->kv_scale_v = device_alloc<float>(sc);
    (void)hipMemset(m->kv_cache_k, 0, kv);
    (void)hipMemset(m->kv_cache_v, 0, kv);
    (void)hipMemset(m->kv_scale_k, 0, sc * sizeof(float));
    (void)hipMemset(m->kv_scale_v, 0, sc * sizeof(float));
}

int default_context(const ModelConfig& c)
{
    const char* env = getenv("TURBO_CTX");
    if (env) return atoi(env);
    const int head_dim = c.n_embd / c.n_head;
    const size_t per_tok = (size_t)c.n_layer * c.n_head_kv * head_dim * 2 + (size_t)c.n_layer * c.n_head_kv * 2 * 4;
    size_t free_b = 0, total_b = 0;
    (void)hipMemGetInfo(&free_b, &total_b);
    const size_t budget = free_b > (512u << 20) ? free_b - (512u << 20) : free_b / 2;
    return (int)std::min<size_t>(8192, budget / std::max<size_t>(per_tok, 1));
}

}  // namespace

bool check_model_dir(const std::string& model_path, std::string& err)
{
    ModelConfig c;
    if (!read_config(model_path, c, err)) return false;
    if (file_size(model_path + "/tok_embd.bin") != (long long)c.n_vocab * c.n_embd * 2)
        return fail(err, "Missing tok_embd.bin (or wrong size)");
    auto norm_ok = [&](const std::string& name) {
        if (file_size(model_path + "/" + name) == (long long)c.n_embd * 4) return true;
        return fail(err, name + " missing or not n_embd floats");
    };
    if (!norm_ok("output_norm.bin")) return false;
    if (!check_tensor(model_path, "output_proj", c.n_vocab, c.n_embd, err)) return false;
    for (int i = 0; i < c.n_layer; i++) {
        const std::string p = "layer." + std::to_string(i) + ".";
        if (!norm_ok(p + "attn_norm.bin") || !norm_ok(p + "ffn_norm.bin")) return false;
        for (int t = 0; t < 7; t++) {
            int M, K;
            tensor_shape(c, t, M, K);
            if (!check_tensor(model_path, p + kTensorNames[t], M, K, err)) return false;
        }
    }
    return true;
}

Model* load_model(const std::string& model_path, int device_id)
{
    // Everything that can be wrong with the directory is found on the host first: a norm that is missing, a tensor
    // whose shape is not its role's, a list that points outside its row would each become a device memory fault in
    // the first forward.  (The reference warns and carries on, engine/model.cpp:203-242.)
    std::string err;
    if (!check_model_dir(model_path, err)) {
        fprintf(stderr, "%s\n", err.c_str());
        return nullptr;
    }
    if (!gpu_ok(hipSetDevice(device_id), "hipSetDevice")) return nullptr;
    Model* m = new Model();
    ModelConfig& c = m->config;
    read_config(model_path, c, err);
    printf("  Config: vocab=%d embd=%d heads=%d/%d layers=%d ff=%d\n", c.n_vocab, c.n_embd, c.n_head, c.n_head_kv,
           c.n_layer, c.n_ff);

    std::vector<uint8_t> buf;
    bool ok = read_file(model_path + "/tok_embd.bin", buf, true) && buf.size() == (size_t)c.n_vocab * c.n_embd * 2;
    if (ok) m->token_embd = upload<int16_t>(buf.data(), buf.size() / 2);
    buf.clear();
    buf.shrink_to_fit();

    auto load_norm = [&](const std::string& name) -> float* {
        std::vector<uint8_t> nb;
        if (!read_file(model_path + "/" + name, nb, true) || nb.size() != (size_t)c.n_embd * 4) {
            fprintf(stderr, "%s missing or wrong size\n", name.c_str());
            ok = false;
            return nullptr;
        }
        return upload<float>(nb.data(), c.n_embd);
    };
    if (ok) m->output_norm = load_norm("output_norm.bin");
    ok = ok && load_compressed(model_path, "output_proj", m->output_proj);

    m->layers.resize(c.n_layer);
    for (auto& L : m->layers) {
        L.attn_norm = L.ffn_norm = nullptr;
        for (CompressedWeight* w : {&L.wq, &L.wk, &L.wv, &L.wo, &L.w_gate, &L.w_up, &L.w_down}) clear_weight(*w);
    }
    for (int i = 0; ok && i < c.n_layer; i++) {
        TransformerLayer& L = m->layers[i];
        const std::string p = "layer." + std::to_string(i) + ".";
        L.attn_norm = load_norm(p + "attn_norm.bin");
        L.ffn_norm = load_norm(p + "ffn_norm.bin");
        CompressedWeight* all[7] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.w_gate, &L.w_up, &L.w_down};
        for (int t = 0; ok && t < 7; t++) ok = load_compressed(model_path, p + kTensorNames[t], *all[t]);
        if (ok && ((i + 1) % 8 == 0 || i == c.n_layer - 1)) printf("  Loaded layer %d/%d\n", i + 1, c.n_layer);
    }
    if (!ok) {                                      // a file changed under the check, or could not be read
        free_model(m);
        return nullptr;
    }
    alloc_kv_cache(m, default_context(c));
    printf("  Context length: %d\n  Model loaded.\n", m->max_seq_len);
    return m;
}

void free_model(Model* model)
{
    if (!model) return;
    if (model->token_embd) (void)hipFree(model->token_embd);
    if (model->output_norm) (void)hipFree(model->output_norm);
    free_weight(model->output_proj);
    for (auto& L : model->layers) {
        if (L.attn_norm) (void)hipFree(L.attn_norm);
        if (L.ffn_norm) (void)hipFree(L.ffn_norm);
        for (CompressedWeight* w : {&L.wq, &L.wk, &L.wv, &L.wo, &L.w_gate, &L.w_up, &L.w_down}) free_weight(*w);
    }
    for (void* p : {(void*)model->kv_cache_k, (void*)model->kv_cache_v, (void*)model->kv_scale_k, (void*)model->kv_scale_v})
        if (p) (void)hipFree(p);
    delete model;
}

// ------------------------------------------------------------ synthetic model
namespace {

// Packs a bf16 matrix resident in HBM with the GPU packer; fills every field of w.
bool pack_on_gpu(const void* w_bf16, int M, int K, CompressedWeight& w)
{
    clear_weight(w);
    const size_t n = (size_t)M * K;
    unsigned long long* d_hist = device_alloc<unsigned long long>(256);
    uint64_t hist[256];
    if (t12_pack_histogram(w_bf16, n, d_hist, nullptr) != T12_OK ||
        !gpu_ok(hipMemcpy(hist, d_hist, sizeof hist, hipMemcpyDeviceToHost), "hist copy")) {
        (void)hipFree(d_hist);
        return false;
    }
    (void)hipFree(d_hist);
    const int be = t12_pack_base_exp(hist);
    w.M = M;
    w.K = K;
    w.base_exp = be;
    w.split_sm = device_alloc<uint8_t>(n);
    w.split_gr = device_alloc<uint8_t>((n + 1) / 2);
    int32_t* cnt = device_alloc<int32_t>(M);
    int32_t* ro = device_alloc<int32_t>(M + 1);
    bool ok = t12_pack_planes(w_bf16, M, K, be, w.split_sm, w.split_gr, cnt, nullptr) == T12_OK &&
              t12_pack_row_offsets(cnt, M, ro, nullptr) == T12_OK;
    int P = 0;
    ok = ok && gpu_ok(hipMemcpy(&P, ro + M, sizeof(int), hipMemcpyDeviceToHost), "P copy");
    (void)hipFree(cnt);
    if (!ok) { (void)hipFree(ro); return false; }
    w.num_patches = P;
    if (P == 0) {
        (void)hipFree(ro);
        return true;
    }
    w.row_offsets = ro;
    w.patch_cols = device_alloc<int32_t>(P);
    w.patch_correct = device_alloc<int16_t>(P);
    w.patch_wrong = device_alloc<int16_t>(P);
    if (t12_pack_escapes(w_bf16, M, K, be, ro, w.patch_cols, w.patch_correct, w.patch_wrong, nullptr) != T12_OK)
        return false;
    std::vector<int32_t> h_ro(M + 1), h_pc(P);
    std::vector<int16_t> h_pv(P);
    ok = gpu_ok(hipMemcpy(h_ro.data(), ro, (M + 1) * 4, hipMemcpyDeviceToHost), "row_off copy") &&
         gpu_ok(hipMemcpy(h_pc.data(), w.patch_cols, (size_t)P * 4, hipMemcpyDeviceToHost), "cols copy") &&
         gpu_ok(hipMemcpy(h_pv.data(), w.patch_correct, (size_t)P * 2, hipMemcpyDeviceToHost), "correct copy");
    if (ok) build_escape_tables(w, h_ro.data(), h_pc.data(), h_pv.data());
    return ok;
}

template <typename T>
bool dump(const std::string& path, const T* dev, size_t count)
{
    std::vector<T> h(count);
    if (count && !gpu_ok(hipMemcpy(h.data(), dev, count * sizeof(T), hipMemcpyDeviceToHost), "download")) return false;
    std::ofstream f(path, std::ios::binary);
    if (f && count) f.write((const char*)h.data(), (std::streamsize)(count * sizeof(T)));
    if (!f) fprintf(stderr, "Cannot write: %s\n", path.c_str());
    return (bool)f;
}

bool save_weight(const std::string& dir, const std::string& prefix, const CompressedWeight& w)
{
    const std::string b = dir + "/" + prefix;
    const size_t n = (size_t)w.M * w.K;
    const size_t P = (size_t)w.num_patches;
    bool ok = dump<uint8_t>(b + ".sm.bin", w.split_sm, n) && dump<uint8_t>(b + ".gr.bin", w.split_gr, (n + 1) / 2);
    if (P > 0) {
        ok = ok && dump<int32_t>(b + ".row_off.bin", w.row_offsets, w.M + 1);
    } else {                                         // the packer always writes M+1 zeros
        std::vector<int32_t> z(w.M + 1, 0);
        std::ofstream f(b + ".row_off.bin", std::ios::binary);
        f.write((const char*)z.data(), (std::streamsize)(z.size() * 4));
        ok = ok && (bool)f;
    }
    ok = ok && dump<int32_t>(b + ".patch_cols.bin", w.patch_cols, P) &&
         dump<int16_t>(b + ".patch_correct.bin", w.patch_correct, P) &&
         dump<int16_t>(b + ".patch_wrong.bin", w.patch_wrong, P);
    std::ofstream d(b + ".dims");
    d << w.M << " " << w.K << " " << w.num_patches << " " << w.base_exp;   // no newline (convert_model.py:133-134)
    return ok && (bool)d;
}

}  // namespace

Model* create_synthetic_model(const ModelConfig& cfg, uint64_t seed, int max_seq_len, float p_outlier)
{
    if (cfg.n_vocab <= 0 || cfg.n_embd <= 0 || cfg.n_head <= 0 || cfg.n_head_kv <= 0 || cfg.n_ff <= 0 ||
        cfg.n_embd % cfg.n_head || cfg.n_head % cfg.n_head_kv)
        return nullptr;
    Model* m = new Model();
    m->config = cfg;
    const int n = cfg.n_embd, ff = cfg.n_ff;
    const int kv = cfg.n_head_kv * (n / cfg.n_head);
    const size_t biggest = std::max({(size_t)cfg.n_vocab * n, (size_t)ff * n});
    uint16_t* stage = device_alloc<uint16_t>(biggest);
    uint64_t s = seed;
    bool ok = true;
    auto make = [&](int M, int K, CompressedWeight& w) {
        ok = ok && t12_synth_normal_bf16(stage, (size_t)M * K, ++s, 0.02f, p_outlier, 8.0f, nullptr) == T12_OK &&
             pack_on_gpu(stage, M, K, w);
    };
    auto ones = [&]() {
        float* d = device_alloc<float>(n);
        ok = ok && t12_fill_f32(d, n, 1.0f, nullptr) == T12_OK;
        return d;
    };
    m->token_embd = device_alloc<int16_t>((size_t)cfg.n_vocab * n);
    ok = ok && t12_synth_normal_bf16(m->token_embd, (size_t)cfg.n_vocab * n, ++s, 0.02f, 0.0f, 0.0f, nullptr) == T12_OK;
    m->output_norm = ones();
    m->layers.resize(cfg.n_layer);
    for (auto& L : m->layers) {
        L.attn_norm = ones();
        L.ffn_norm = ones();
        make(n, n, L.wq);
        make(kv, n, L.wk);
        make(kv, n, L.wv);
        make(n, n, L.wo);
        make(ff, n, L.w_gate);
        make(ff, n, L.w_up);
        make(n, ff, L.w_down);
    }
    make(cfg.n_vocab, n, m->output_proj);
    ok = ok && gpu_ok(hipDeviceSynchronize(), "synthetic model");
    (void)hipFree(stage);
    if (!ok) {
        free_model(m);
        return nullptr;
    }
    alloc_kv_cache(m, max_seq_len > 0 ? max_seq_len : default_context(cfg));
    return m;
}

bool save_model(const Model* m, const std::string& dir)
{
    const ModelConfig& c = m->config;
    struct { int32_t v[7]; float theta, eps; } raw = {{c.n_vocab, c.n_embd, c.n_head, c.n_head_kv, c.n_layer, c.n_ff,
                                                       c.n_ctx}, c.rope_theta, c.rms_norm_eps};
    {
        std::ofstream f(dir + "/config.bin", std::ios::binary);
        if (!f) {
            fprintf(stderr, "Cannot write: %s/config.bin (the directory must exist)\n", dir.c_str());
            return false;
        }
        f.write((const char*)&raw, sizeof raw);
    }
    if (c.rope_scaling[0] > 0.0f) {
        std::ofstream f(dir + "/rope_scaling.bin", std::ios::binary);
        if (!f) return false;
        f.write((const char*)c.rope_scaling, sizeof c.rope_scaling);
    }
    bool ok = dump<int16_t>(dir + "/tok_embd.bin", m->token_embd, (size_t)c.n_vocab * c.n_embd) &&
              dump<float>(dir + "/output_norm.bin", m->output_norm, c.n_embd) &&
              save_weight(dir, "output_proj", m->output_proj);
    for (int i = 0; ok && i < c.n_layer; i++) {
        const TransformerLayer& L = m->layers[i];
        const std::string p = "layer." + std::to_string(i) + ".";
        ok = dump<float>(dir + "/" + p + "attn_norm.bin", L.attn_norm, c.n_embd) &&
             dump<float>(dir + "/" + p + "ffn_norm.bin", L.ffn_norm, c.n_embd) && save_weight(dir, p + "wq", L.wq) &&
             save_weight(dir, p + "wk", L.wk) && save_weight(dir, p + "wv", L.wv) && save_weight(dir, p + "wo", L.wo) &&
             save_weight(dir, p + "w_gate", L.w_gate) && save_weight(dir, p + "w_up", L.w_up) &&
             save_weight(dir, p + "w_down", L.w_down);
    }
    return ok;
}
