/*
 * CPU oracle for the split-12 path.  TEST INFRASTRUCTURE ONLY: this file is the
 * checker that tests, the smoke check and the benchmark's cpu_baseline leg
 * compare the HIP kernels against.  Nothing in the shipped library links,
 * loads or calls it.
 *
 * Every function restates, in plain C, the algorithm of the reference file
 * cited above it.  Pinning (what keeps each function honest):
 *   t12o_find_base_exp, t12o_pack  byte equality with the reference C packer
 *                                  (oracle/_ref, built from split12_pack.c) on the
 *                                  committed golden fixtures + brute-force window
 *                                  search on tiny inputs
 *   t12o_decode                    lossless identity decode(pack(W)) == W and
 *                                  patch_wrong == unpatched decode at escapes
 *   t12o_escape_tables             brute-force recomputation from the CSR lists
 *   t12o_gemv / t12o_gemm          numpy float64 matmul on the decoded weights
 *
 * Build: see oracle/Makefile (gcc -O3 -fopenmp -shared).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ helpers */
static inline float bf16_bits_to_f32(uint16_t b)
{
    union { uint32_t u; float f; } c;
    c.u = (uint32_t)b << 16;
    return c.f;
}

static inline uint16_t t12o_decode_one(uint8_t sm, uint32_t g, int base_exp)
{
    /* decode rule: decompress_v2.hip:192, nvidia_kernels.cu:545-546,
     * split12_gemm.cuh:52-57 -- exponent = base_exp + group, truncated to 16 bits */
    return (uint16_t)(((uint16_t)(sm >> 7) << 15) |
                      (uint16_t)((uint32_t)(base_exp + (int)g) << 7) |
                      (uint16_t)(sm & 0x7F));
}

static inline uint32_t nibble_at(const uint8_t *gr, int64_t i)
{
    /* flat element index i; even -> low nibble, odd -> high (split12_pack.c:87-90) */
    uint8_t b = gr[i >> 1];
    return (i & 1) ? (uint32_t)(b >> 4) : (uint32_t)(b & 0xF);
}

/* threads the parallel loops below use from now on (n < 1: back to the OpenMP default) */
void t12o_set_num_threads(int n)
{
    omp_set_num_threads(n >= 1 ? n : omp_get_num_procs());
}

int t12o_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* --------------------------------------------------------- find_base_exp
 * Follows split12_pack.c:18-37: 256-bin histogram of the exponent byte, then
 * the 15-wide window with the largest population; strict '>' so the earliest
 * window wins ties; result is window_start - 1 (so -1 for empty/all-zero). */
int t12o_find_base_exp(const uint16_t *w, int64_t count)
{
    int64_t hist[256];
    memset(hist, 0, sizeof hist);
    for (int64_t i = 0; i < count; i++)
        hist[(w[i] >> 7) & 0xFF]++;

    int64_t run = 0;
    for (int j = 0; j < 15; j++) run += hist[j];
    int64_t best = 0;
    int best_start = 0;
    for (int s = 0; s <= 241; s++) {
        if (s > 0) run += hist[s + 14] - hist[s - 1];
        if (run > best) { best = run; best_start = s; }
    }
    return best_start - 1;
}

/* ------------------------------------------------------------------- pack
 * Follows split12_pack.c:47-128.  Outputs:
 *   sm[i]      = sign<<7 | mantissa7
 *   gr[i/2]    nibble (low = even i, high = odd i) = exponent - base_exp if that
 *              lies in 1..15 and the exponent itself is a valid byte, else 0
 *   row_off    CSR pointers over escapes, cols ascending inside a row
 *   correct    original bf16 bits;  wrong = sign<<15 | (u16)(base_exp<<7) | mant
 * Returns the number of escapes.  Patch arrays must hold at least that many
 * entries (t12o_count_escapes gives the exact figure). */
static inline int group_of(uint32_t e, int base_exp)
{
    int g = (int)e - base_exp;
    return (g >= 1 && g <= 15) ? g : 0;
}

int64_t t12o_count_escapes(const uint16_t *w, int64_t count, int base_exp)
{
    int64_t n = 0;
    for (int64_t i = 0; i < count; i++)
        n += group_of((w[i] >> 7) & 0xFF, base_exp) == 0;
    return n;
}

int64_t t12o_pack(const uint16_t *w, int M, int K, int base_exp,
                  uint8_t *sm, uint8_t *gr, int32_t *row_off,
                  int32_t *cols, int16_t *correct, int16_t *wrong)
{
    const int64_t count = (int64_t)M * K;
    memset(gr, 0, (size_t)((count + 1) / 2));
    int64_t p = 0;
    row_off[0] = 0;
    for (int r = 0; r < M; r++) {
        for (int c = 0; c < K; c++) {
            const int64_t i = (int64_t)r * K + c;
            const uint16_t v = w[i];
            const uint8_t s = (uint8_t)(((v >> 15) << 7) | (v & 0x7F));
            const int g = group_of((v >> 7) & 0xFF, base_exp);
            sm[i] = s;
            gr[i >> 1] |= (uint8_t)(g << (4 * (int)(i & 1)));
            if (g == 0) {
                cols[p] = c;
                correct[p] = (int16_t)v;
                wrong[p] = (int16_t)t12o_decode_one(s, 0, base_exp);
                p++;
            }
        }
        row_off[r + 1] = (int32_t)p;
    }
    return p;
}

/* ----------------------------------------------------------------- decode
 * The reference ships no CPU decoder; this is the inverse of pack_split12 using
 * the rule every GPU kernel of the reference states (see t12o_decode_one).
 * patched != 0: escapes (group 0) take patch_correct -> lossless.
 * patched == 0: semantics of nv_decode_split12_to_bf16 (nvidia_kernels.cu:533-548):
 *               escapes come out as the "wrong" value. */
void t12o_decode(const uint8_t *sm, const uint8_t *gr, int base_exp, int M, int K,
                 const int32_t *row_off, const int32_t *cols, const int16_t *correct,
                 int patched, uint16_t *out)
{
    const int64_t count = (int64_t)M * K;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < count; i++)
        out[i] = t12o_decode_one(sm[i], nibble_at(gr, i), base_exp);
    if (patched && row_off) {
        for (int r = 0; r < M; r++)
            for (int32_t p = row_off[r]; p < row_off[r + 1]; p++)
                out[(int64_t)r * K + cols[p]] = (uint16_t)correct[p];
    }
}

/* ---------------------------------------------------------- escape tables
 * Follows engine/model.cpp:86-160 (WG = 256): counts[r*256 + col%256],
 * row_base[r] = escapes before row r, esc_vals ordered by (row, col%256,
 * ascending col); nonempty = rows holding at least one escape.
 * Returns the number of non-empty rows. */
int t12o_escape_tables(int M, const int32_t *row_off, const int32_t *cols,
                       const int16_t *correct, int32_t *row_base, uint8_t *counts_u8,
                       int16_t *esc_vals, int32_t *nonempty)
{
    const int WG = 256;
    int32_t *cnt = (int32_t *)calloc((size_t)M * WG, sizeof(int32_t));
    int32_t *off = (int32_t *)malloc((size_t)M * WG * sizeof(int32_t));
    for (int r = 0; r < M; r++)
        for (int32_t p = row_off[r]; p < row_off[r + 1]; p++)
            cnt[(size_t)r * WG + cols[p] % WG]++;
    int32_t total = 0;
    int nne = 0;
    for (int r = 0; r < M; r++) {
        row_base[r] = total;
        for (int t = 0; t < WG; t++) {
            off[(size_t)r * WG + t] = total;
            total += cnt[(size_t)r * WG + t];
        }
        if (row_off[r + 1] > row_off[r]) nonempty[nne++] = r;
    }
    for (int r = 0; r < M; r++)
        for (int32_t p = row_off[r]; p < row_off[r + 1]; p++)
            esc_vals[off[(size_t)r * WG + cols[p] % WG]++] = correct[p];
    if (counts_u8)
        for (size_t i = 0; i < (size_t)M * WG; i++) counts_u8[i] = (uint8_t)cnt[i];
    free(cnt);
    free(off);
    return nne;
}

/* ------------------------------------------------------------ GEMV / GEMM
 * out[b*out_stride + m] = sum_k f32(dec(W[m,k])) * f32(X[b*x_stride + k]), fp32
 * accumulate in ascending k.  Semantics: decompress_v2.hip:148-227 (matvec) and
 * split12_gemm.cuh:273-284 (output layout), with escapes taken from the CSR list
 * (exact) when row_off != NULL, or left as the "wrong" value when NULL.
 * The decode is fused (no bf16 matrix is materialised), rows run in parallel:
 * this is also the timed CPU baseline. */
void t12o_gemm(const uint8_t *sm, const uint8_t *gr, int base_exp, int M, int K,
               const int32_t *row_off, const int32_t *cols, const int16_t *correct,
               const uint16_t *X, int x_stride, int B, float *out, int out_stride)
{
#pragma omp parallel
    {
        float *wrow = (float *)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (int m = 0; m < M; m++) {
            const int64_t base = (int64_t)m * K;
            for (int k = 0; k < K; k++)
                wrow[k] = bf16_bits_to_f32(
                    t12o_decode_one(sm[base + k], nibble_at(gr, base + k), base_exp));
            if (row_off)
                for (int32_t p = row_off[m]; p < row_off[m + 1]; p++)
                    wrow[cols[p]] = bf16_bits_to_f32((uint16_t)correct[p]);
            for (int b = 0; b < B; b++) {
                const uint16_t *x = X + (int64_t)b * x_stride;
                float acc = 0.0f;
                for (int k = 0; k < K; k++)
                    acc += wrow[k] * bf16_bits_to_f32(x[k]);
                out[(int64_t)b * out_stride + m] = acc;
            }
        }
        free(wrow);
    }
}

void t12o_gemv(const uint8_t *sm, const uint8_t *gr, int base_exp, int M, int K,
               const int32_t *row_off, const int32_t *cols, const int16_t *correct,
               const uint16_t *x, float *out)
{
    t12o_gemm(sm, gr, base_exp, M, K, row_off, cols, correct, x, K, 1, out, M);
}

/* Patch correction as the reference's B=1 path applies it after an unpatched
 * matvec (decompress_v2.hip:78-99):
 *   out[m] += sum_p (f32(correct_p) - f32(wrong_p)) * f32(x[col_p])        */
void t12o_apply_patches(const int32_t *row_off, const int32_t *cols,
                        const int16_t *correct, const int16_t *wrong,
                        const uint16_t *x, float *out, int M)
{
    for (int m = 0; m < M; m++) {
        float c = 0.0f;
        for (int32_t p = row_off[m]; p < row_off[m + 1]; p++)
            c += (bf16_bits_to_f32((uint16_t)correct[p]) - bf16_bits_to_f32((uint16_t)wrong[p])) *
                 bf16_bits_to_f32(x[cols[p]]);
        if (c != 0.0f) out[m] += c;
    }
}
