/*
 * CPU restatement of fastvideo-rs's host-math SDPA / block-causal / VSA path.
 * TEST INFRASTRUCTURE ONLY: the parity checker and the timed CPU baseline.
 * See fv_oracle.h for the reference citations and how each function is pinned.
 *
 * Build: gcc -O3 -ffp-contract=off -fopenmp -shared -fPIC (see Makefile).
 * -ffp-contract=off keeps mul and add separate, as the Rust reference does
 * (rustc never contracts a*b+c); vectorising the j loops does not reorder any
 * accumulation, so -O3 and -O2 give the same bits.
 */
#include "fv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define NEG_INF (-INFINITY)

/* ---- bf16 ---------------------------------------------------------------- */

static inline uint32_t f2u(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    return u;
}
static inline float u2f(uint32_t u) {
    float x;
    memcpy(&x, &u, 4);
    return x;
}

/* C/rt/kernels/core.cu:6-15 (== half::bf16::from_f32, C/rt/quant.rs:60-62):
 * round to nearest even; NaN stays a quiet NaN; overflow rounds to inf. */
uint16_t fvo_bf16_rne_bits(float x) {
    uint32_t u = f2u(x);
    if ((u & 0x7F800000u) == 0x7F800000u) {
        uint32_t h = u >> 16;
        if (u & 0x007FFFFFu) h |= 0x0040u;
        return (uint16_t)h;
    }
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float fvo_bf16_round(float x) { return u2f(((uint32_t)fvo_bf16_rne_bits(x)) << 16); }

void fvo_quantize_bf16(const float* x, float* y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = fvo_bf16_round(x[i]);
}
void fvo_to_bf16_bits(const float* x, uint16_t* y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = fvo_bf16_rne_bits(x[i]);
}
void fvo_from_bf16_bits(const uint16_t* x, float* y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = u2f(((uint32_t)x[i]) << 16);
}

/* ---- host tensor ops ------------------------------------------------------- */

/* C/rt/tensor.rs:1692-1700: for i, for t, row[j] += a[i,t] * b[t,j]. */
static void matmul_one(const float* a, const float* b, float* o, size_t m, size_t k, size_t n) {
    for (size_t i = 0; i < m; i++) {
        float* row = o + i * n;
        for (size_t j = 0; j < n; j++) row[j] = 0.0f;
        for (size_t t = 0; t < k; t++) {
            const float av = a[i * k + t];
            const float* br = b + t * n;
            for (size_t j = 0; j < n; j++) row[j] += av * br[j];
        }
    }
}

void fvo_matmul(const float* a, const float* b, float* out, size_t batch, size_t m, size_t k,
                size_t n, int threads) {
    if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1)
    for (long bi = 0; bi < (long)batch; bi++)
        matmul_one(a + (size_t)bi * m * k, b + (size_t)bi * k * n, out + (size_t)bi * m * n, m, k, n);
}

/* C/rt/ops.rs:2183-2190 */
static void softmax_row(const float* row, float* o, size_t width) {
    float m = NEG_INF;
    for (size_t j = 0; j < width; j++) m = fmaxf(m, row[j]);
    float sum = 0.0f;
    for (size_t j = 0; j < width; j++) {
        o[j] = expf(row[j] - m);
        sum += o[j];
    }
    const float inv = 1.0f / sum;
    for (size_t j = 0; j < width; j++) o[j] *= inv;
}

void fvo_softmax_last(const float* x, float* out, size_t rows, size_t width) {
    for (size_t r = 0; r < rows; r++) softmax_row(x + r * width, out + r * width, width);
}

static void transpose_one(const float* x, float* y, size_t r, size_t c) {
    for (size_t i = 0; i < r; i++)
        for (size_t j = 0; j < c; j++) y[j * r + i] = x[i * c + j];
}

/* C/rt/sdpa.rs:328-342, op by op on whole-batch buffers. */
void fvo_sdpa_composed(const float* q, const float* k, const float* v, const float* mask,
                       float* out, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                       int threads) {
    /* calloc: sizes of zero stay valid, and the buffers start defined */
    float* kt = (float*)calloc(bh * d * sk + 1, sizeof(float));
    float* scores = (float*)calloc(bh * sq * sk + 1, sizeof(float));
    float* probs = (float*)calloc(bh * sq * sk + 1, sizeof(float));
    if (!kt || !scores || !probs) {
        free(kt);
        free(scores);
        free(probs);
        return;
    }
    for (size_t b = 0; b < bh; b++) transpose_one(k + b * sk * d, kt + b * d * sk, sk, d);
    fvo_matmul(q, kt, scores, bh, sq, d, sk, threads);           /* q.matmul(k^T)   */
    for (size_t i = 0; i < bh * sq * sk; i++) scores[i] = scores[i] * scale; /* mul_scalar */
    if (mask)                                                     /* scores.add(m)   */
        for (size_t b = 0; b < bh; b++)
            for (size_t i = 0; i < sq * sk; i++)
                scores[b * sq * sk + i] = scores[b * sq * sk + i] + mask[i];
    fvo_softmax_last(scores, probs, bh * sq, sk);                 /* softmax(-1)     */
    fvo_matmul(probs, v, out, bh, sq, sk, d, threads);            /* .matmul(v)      */
    free(kt);
    free(scores);
    free(probs);
}

static inline int bc_allows(const int64_t* bc, size_t q, size_t k) {
    return fvo_block_causal_allows((size_t)bc[0], (size_t)bc[1], (size_t)bc[2], q, k);
}

void fvo_sdpa_composed_rows(const float* q, const float* k, const float* v,
                            const int64_t* mask_bc, const int64_t* rows, size_t nrows,
                            float* out, size_t bh, size_t sq, size_t sk, size_t d,
                            float scale, int threads) {
    if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1)
    for (long b = 0; b < (long)bh; b++) {
        float* kt = (float*)malloc(sizeof(float) * d * sk);
        float* s = (float*)malloc(sizeof(float) * sk);
        float* p = (float*)malloc(sizeof(float) * sk);
        transpose_one(k + (size_t)b * sk * d, kt, sk, d);
        const float* vb = v + (size_t)b * sk * d;
        for (size_t r = 0; r < nrows; r++) {
            const size_t i = (size_t)rows[r];
            const float* qi = q + ((size_t)b * sq + i) * d;
            for (size_t j = 0; j < sk; j++) s[j] = 0.0f;
            for (size_t t = 0; t < d; t++) {
                const float av = qi[t];
                const float* br = kt + t * sk;
                for (size_t j = 0; j < sk; j++) s[j] += av * br[j];
            }
            for (size_t j = 0; j < sk; j++) s[j] = s[j] * scale;
            if (mask_bc)
                for (size_t j = 0; j < sk; j++) s[j] = s[j] + (bc_allows(mask_bc, i, j) ? 0.0f : -1e9f);
            softmax_row(s, p, sk);
            float* o = out + ((size_t)b * nrows + r) * d;
            for (size_t j = 0; j < d; j++) o[j] = 0.0f;
            for (size_t t = 0; t < sk; t++) {
                const float av = p[t];
                const float* vr = vb + t * d;
                for (size_t j = 0; j < d; j++) o[j] += av * vr[j];
            }
        }
        free(kt);
        free(s);
        free(p);
    }
}

/* ---- f64 checker ----------------------------------------------------------- */

void fvo_sdpa_f64_rows(const float* q, const float* k, const float* v, const int64_t* mask_bc,
                       const int64_t* rows, size_t nrows, float* out, size_t bh, size_t sq,
                       size_t sk, size_t d, double scale, int threads) {
    if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1) collapse(2)
    for (long b = 0; b < (long)bh; b++) {
        for (long r = 0; r < (long)nrows; r++) {
            const size_t i = rows ? (size_t)rows[r] : (size_t)r;
            double* p = (double*)malloc(sizeof(double) * sk);
            double* acc = (double*)calloc(d, sizeof(double));
            const float* qi = q + ((size_t)b * sq + i) * d;
            double mx = -INFINITY;
            for (size_t j = 0; j < sk; j++) {
                if (mask_bc && !bc_allows(mask_bc, i, j)) {
                    p[j] = -INFINITY;
                } else {
                    const float* kj = k + ((size_t)b * sk + j) * d;
                    double dot = 0.0;
                    for (size_t c = 0; c < d; c++) dot += (double)qi[c] * (double)kj[c];
                    p[j] = dot * scale;
                }
                if (p[j] > mx) mx = p[j];
            }
            double z = 0.0;
            for (size_t j = 0; j < sk; j++) {
                p[j] = exp(p[j] - mx);
                z += p[j];
            }
            for (size_t j = 0; j < sk; j++) {
                if (p[j] == 0.0) continue;
                const float* vj = v + ((size_t)b * sk + j) * d;
                for (size_t c = 0; c < d; c++) acc[c] += p[j] * (double)vj[c];
            }
            float* o = out + ((size_t)b * nrows + (size_t)r) * d;
            for (size_t c = 0; c < d; c++) o[c] = (float)(acc[c] / z);
            free(p);
            free(acc);
        }
    }
}

void fvo_sdpa_f64(const float* q, const float* k, const float* v, const int64_t* mask_bc,
                  float* out, size_t bh, size_t sq, size_t sk, size_t d, double scale,
                  int threads) {
    fvo_sdpa_f64_rows(q, k, v, mask_bc, NULL, sq, out, bh, sq, sk, d, scale, threads);
}

/* ---- block-causal mask ----------------------------------------------------- */

/* C/rt/attn.rs:449-453 */
int fvo_block_causal_allows(size_t block_tokens, size_t window, size_t sink, size_t q, size_t k) {
    const size_t bt = block_tokens > 1 ? block_tokens : 1;
    const size_t tq = q / bt, tk = k / bt;
    return (tk <= tq && (window == 0 || tq - tk < window)) || tk < sink;
}

/* C/rt/attn.rs:456-466 */
void fvo_block_causal_dense_mask(size_t block_tokens, size_t window, size_t sink, size_t sq,
                                 size_t sk, float* mask) {
    for (size_t q = 0; q < sq; q++)
        for (size_t k = 0; k < sk; k++)
            mask[q * sk + k] = fvo_block_causal_allows(block_tokens, window, sink, q, k) ? 0.0f : -1e9f;
}

/* C/rt/attn.rs:630-645 */
int fvo_block_causal_for(size_t num_frames_per_block, int64_t local_attn_size,
                         size_t frame_tokens, size_t* out3) {
    const size_t fpb = num_frames_per_block > 1 ? num_frames_per_block : 1;
    size_t window;
    if (local_attn_size < 0) {
        window = 0;
    } else if (local_attn_size > 0 && (size_t)local_attn_size % fpb == 0) {
        window = (size_t)local_attn_size / fpb;
    } else {
        return 0;
    }
    out3[0] = fpb * frame_tokens;
    out3[1] = window;
    out3[2] = 0;
    return 1;
}

/* M/wan/family.rs:80-111 */
void fvo_causal_temporal_mask(const size_t patch[3], size_t num_frames_per_block,
                              int64_t local_attn_size, size_t frames, size_t height,
                              size_t width, float* mask) {
    const size_t pt = patch[0] > 1 ? patch[0] : 1;
    const size_t ph = patch[1] > 1 ? patch[1] : 1;
    const size_t pw = patch[2] > 1 ? patch[2] : 1;
    const size_t tf = frames / pt, hf = height / ph, wf = width / pw;
    const size_t seq = tf * hf * wf;
    const size_t frame_tokens = hf * wf;
    size_t block = (num_frames_per_block > 1 ? num_frames_per_block : 1) * frame_tokens;
    if (block < 1) block = 1;
    const int has_window = local_attn_size >= 0;
    const size_t w = has_window ? (size_t)local_attn_size * frame_tokens : 0;
    for (size_t q = 0; q < seq; q++) {
        const size_t end = (q / block + 1) * block;
        for (size_t k = 0; k < seq; k++) {
            const int ok = (k < end && (!has_window || k + w >= end)) || k == q;
            mask[q * seq + k] = ok ? 0.0f : -1e9f;
        }
    }
}

/* ---- VSA geometry ------------------------------------------------------------ */

/* C/rt/vsa.rs:34-37 */
size_t fvo_topk_for(double sparsity, size_t num_tiles) {
    const double keep_f = ceil((1.0 - sparsity) * (double)num_tiles);
    size_t keep = keep_f <= 0.0 ? 0 : (size_t)keep_f; /* `as usize` saturates at 0 */
    const size_t hi = num_tiles > 1 ? num_tiles : 1;
    if (keep < 1) keep = 1;
    if (keep > hi) keep = hi;
    return keep;
}

/* C/rt/vsa.rs:62-109 */
int fvo_tile_plan(size_t t, size_t h, size_t w, size_t dims_out[5], int32_t* slot_src,
                  uint32_t* token_slot, uint32_t* block_sizes) {
    if (t == 0 || h == 0 || w == 0) return -1;
    const size_t ts = 4, hs = 4, ws = 4, te = 64;
    const size_t nt = (t + ts - 1) / ts, nh = (h + hs - 1) / hs, nw = (w + ws - 1) / ws;
    const size_t num_tiles = nt * nh * nw, seq = t * h * w, padded = num_tiles * te;
    if (dims_out) {
        dims_out[0] = nt;
        dims_out[1] = nh;
        dims_out[2] = nw;
        dims_out[3] = seq;
        dims_out[4] = padded;
    }
    if (!slot_src || !token_slot || !block_sizes) return 0;
    for (size_t i = 0; i < padded; i++) slot_src[i] = -1;
    for (size_t i = 0; i < seq; i++) token_slot[i] = 0;
    size_t tile = 0;
    for (size_t tt = 0; tt < nt; tt++)
        for (size_t hh = 0; hh < nh; hh++)
            for (size_t ww = 0; ww < nw; ww++) {
                size_t slot = tile * te;
                const size_t z1 = (tt + 1) * ts < t ? (tt + 1) * ts : t;
                const size_t y1 = (hh + 1) * hs < h ? (hh + 1) * hs : h;
                const size_t x1 = (ww + 1) * ws < w ? (ww + 1) * ws : w;
                for (size_t z = tt * ts; z < z1; z++)
                    for (size_t y = hh * hs; y < y1; y++)
                        for (size_t x = ww * ws; x < x1; x++) {
                            const size_t token = (z * h + y) * w + x;
                            slot_src[slot] = (int32_t)token;
                            token_slot[token] = (uint32_t)slot;
                            slot++;
                        }
                block_sizes[tile] = (uint32_t)(slot - tile * te);
                tile++;
            }
    return 0;
}

/* ---- top-k --------------------------------------------------------------------- */

/* C/rt/kernels/core.cu:576-579 */
uint32_t fvo_sortable(float x) {
    const uint32_t u = f2u(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

static int cmp_u32_desc(const void* a, const void* b) {
    const uint32_t x = *(const uint32_t*)a, y = *(const uint32_t*)b;
    return x < y ? 1 : (x > y ? -1 : 0);
}

/* C/rt/kernels/core.cu:580-618: T = largest threshold with count(key >= T) >= k,
 * i.e. the k-th largest key; emit key > T ascending, then key == T ascending. */
void fvo_topk_device_order(const float* scores, uint32_t* out, size_t rows, size_t n, size_t k) {
    uint32_t* keys = (uint32_t*)malloc(sizeof(uint32_t) * (n ? n : 1));
    uint32_t* sorted = (uint32_t*)malloc(sizeof(uint32_t) * (n ? n : 1));
    for (size_t r = 0; r < rows; r++) {
        const float* s = scores + r * n;
        for (size_t i = 0; i < n; i++) sorted[i] = keys[i] = fvo_sortable(s[i]);
        qsort(sorted, n, sizeof(uint32_t), cmp_u32_desc);
        /* k > n: count(key >= 0) = n < k for every T, the bisection ends at T = 0 */
        const uint32_t thr = (k >= 1 && k <= n) ? sorted[k - 1] : 0u;
        uint32_t* dst = out + r * k;
        size_t written = 0;
        for (size_t i = 0; i < n && written < k; i++)
            if (keys[i] > thr) dst[written++] = (uint32_t)i;
        for (size_t i = 0; i < n && written < k; i++)
            if (keys[i] == thr) dst[written++] = (uint32_t)i;
        for (; written < k; written++) dst[written] = 0u;
    }
    free(keys);
    free(sorted);
}

typedef struct {
    uint32_t key;
    uint32_t idx;
} key_idx;

static int cmp_key_desc_idx_asc(const void* a, const void* b) {
    const key_idx* x = (const key_idx*)a;
    const key_idx* y = (const key_idx*)b;
    if (x->key != y->key) return x->key < y->key ? 1 : -1;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);
}

/* C/rt/vsa.rs:203-212: sort by (score descending under total_cmp, index
 * ascending); fvo_sortable is monotone in total_cmp's order. */
void fvo_topk_host_order(const float* scores, uint32_t* out, size_t rows, size_t n, size_t k) {
    key_idx* order = (key_idx*)malloc(sizeof(key_idx) * (n ? n : 1));
    for (size_t r = 0; r < rows; r++) {
        const float* s = scores + r * n;
        for (size_t i = 0; i < n; i++) {
            order[i].key = fvo_sortable(s[i]);
            order[i].idx = (uint32_t)i;
        }
        qsort(order, n, sizeof(key_idx), cmp_key_desc_idx_asc);
        for (size_t i = 0; i < k; i++) out[r * k + i] = i < n ? order[i].idx : 0u;
    }
    free(order);
}

/* ---- VSA stages ---------------------------------------------------------------- */

/* C/rt/kernels/core.cu:550-570 */
void fvo_vsa_tile_mean(const float* x, const int32_t* slot_src, const uint32_t* block_sizes,
                       float* out, size_t bh, size_t seq, size_t dim, size_t nb, int round16) {
    for (size_t b = 0; b < bh; b++)
        for (size_t tile = 0; tile < nb; tile++) {
            const uint32_t n = block_sizes[tile];
            for (size_t d = 0; d < dim; d++) {
                float acc = 0.0f;
                for (uint32_t j = 0; j < n; j++) {
                    const size_t tok = (size_t)slot_src[tile * 64 + j];
                    float val = x[(b * seq + tok) * dim + d];
                    if (round16) val = fvo_bf16_round(val);
                    acc += val;
                }
                out[(b * nb + tile) * dim + d] = n > 0 ? acc / (float)n : 0.0f;
            }
        }
}

/* C/rt/kernels/core.cu:803-835 */
void fvo_vsa_combine(const float* sparse, const float* coarse, const float* gate, const int32_t* slot_src,
                     float* out, size_t bh, size_t seq, size_t dim, size_t nb, size_t q_base,
                     size_t q_tiles, int round16) {
    for (size_t b = 0; b < bh; b++)
        for (size_t g = 0; g < q_tiles; g++) {
            const size_t tile = q_base + g;
            if (tile >= nb) continue;
            for (size_t slot = 0; slot < 64; slot++) {
                const int32_t src = slot_src[tile * 64 + slot];
                if (src < 0) continue;
                const float* sp = sparse + ((b * q_tiles + g) * 64 + slot) * dim;
                const float* co = coarse + (b * nb + tile) * dim;
                const float* ga = gate ? gate + (b * seq + (size_t)src) * dim : NULL;
                float* ob = out + (b * seq + (size_t)src) * dim;
                for (size_t d = 0; d < dim; d++) {
                    if (round16) {
                        const float c = fvo_bf16_round(co[d]);
                        const float prod = ga ? c * fvo_bf16_round(ga[d]) : c;
                        const float p = ga ? fvo_bf16_round(prod) : c;
                        const float sum = fvo_bf16_round(sp[d]) + p;
                        ob[d] = fvo_bf16_round(sum);
                    } else {
                        const float prod = co[d] * (ga ? ga[d] : 1.0f);
                        ob[d] = prod + sp[d];
                    }
                }
            }
        }
}

/* C/rt/vsa.rs:185-189: the score of (query tile, key tile) is the f64 dot of the two tile means, d ascending,
 * times f64(scale), cast to f32. The sum starts from -0.0, the identity of Rust's `Sum for f64` at the reference's
 * pinned toolchain (>= 1.88): a dot whose every product is -0.0 stays -0.0, which total_cmp orders below +0.0. */
void fvo_vsa_coarse_scores(const float* qc, const float* kc, float* scores, size_t bh, size_t nb,
                           size_t dim, float scale) {
    for (size_t b = 0; b < bh; b++)
        for (size_t qt = 0; qt < nb; qt++)
            for (size_t kt = 0; kt < nb; kt++) {
                const float* a = qc + (b * nb + qt) * dim;
                const float* c = kc + (b * nb + kt) * dim;
                double dot = -0.0;
                for (size_t d = 0; d < dim; d++) dot += (double)a[d] * (double)c[d];
                scores[(b * nb + qt) * nb + kt] = (float)(dot * (double)scale);
            }
}

/* C/rt/vsa.rs:116-262 */
int fvo_vsa_attention_host(const float* q, const float* k, const float* v, const float* gate,
                           const int32_t* slot_src, const uint32_t* block_sizes, size_t seq,
                           size_t nb, size_t topk, size_t b, size_t heads, size_t dim,
                           float scale, float* out, uint32_t* selected_out) {
    const size_t TE = 64;
    if (topk < 1) topk = 1;
    if (topk > nb) topk = nb;
    const size_t want = b * heads * seq * dim;
    for (size_t i = 0; i < want; i++) out[i] = 0.0f;
    float* qc = (float*)malloc(sizeof(float) * nb * dim);
    float* kc = (float*)malloc(sizeof(float) * nb * dim);
    float* vc = (float*)malloc(sizeof(float) * nb * dim);
    float* coarse = (float*)malloc(sizeof(float) * nb * dim);
    float* scores = (float*)malloc(sizeof(float) * nb * nb);
    double* exps = (double*)malloc(sizeof(double) * nb);
    uint32_t* selected = (uint32_t*)malloc(sizeof(uint32_t) * nb * topk);
    double* acc = (double*)malloc(sizeof(double) * dim);

    for (size_t bh = 0; bh < b * heads; bh++) {
        const size_t base = bh * seq * dim;
        /* 1. tile means (vsa.rs:151-176) */
        memset(qc, 0, sizeof(float) * nb * dim);
        memset(kc, 0, sizeof(float) * nb * dim);
        memset(vc, 0, sizeof(float) * nb * dim);
        for (size_t tile = 0; tile < nb; tile++) {
            const float n = (float)block_sizes[tile];
            if (n == 0.0f) continue;
            for (size_t slot = tile * TE; slot < tile * TE + block_sizes[tile]; slot++) {
                const size_t token = (size_t)slot_src[slot];
                for (size_t d = 0; d < dim; d++) {
                    qc[tile * dim + d] += q[base + token * dim + d];
                    kc[tile * dim + d] += k[base + token * dim + d];
                    vc[tile * dim + d] += v[base + token * dim + d];
                }
            }
            for (size_t d = 0; d < dim; d++) {
                qc[tile * dim + d] /= n;
                kc[tile * dim + d] /= n;
                vc[tile * dim + d] /= n;
            }
        }
        /* 2. coarse attention over tiles, f64 (vsa.rs:179-199) */
        memset(coarse, 0, sizeof(float) * nb * dim);
        for (size_t qt = 0; qt < nb; qt++) {
            float* s = scores + qt * nb;
            for (size_t kt = 0; kt < nb; kt++) {
                double dot = -0.0;   /* the identity of Rust's f64 Sum */
                for (size_t d = 0; d < dim; d++)
                    dot += (double)qc[qt * dim + d] * (double)kc[kt * dim + d];
                s[kt] = (float)(dot * (double)scale);
            }
            float m = NEG_INF;
            for (size_t kt = 0; kt < nb; kt++) m = fmaxf(m, s[kt]);
            double z = 0.0;
            for (size_t kt = 0; kt < nb; kt++) {
                exps[kt] = exp((double)(s[kt] - m));
                z += exps[kt];
            }
            for (size_t kt = 0; kt < nb; kt++) {
                const double wgt = exps[kt] / z;
                for (size_t d = 0; d < dim; d++)
                    coarse[qt * dim + d] += (float)(wgt * (double)vc[kt * dim + d]);
            }
        }
        /* 3. top-k tiles per query tile (vsa.rs:203-212) */
        fvo_topk_host_order(scores, selected, nb, nb, topk);
        if (selected_out) memcpy(selected_out + bh * nb * topk, selected, sizeof(uint32_t) * nb * topk);
        /* 4. fine attention inside the selected tiles, then combine (vsa.rs:215-258) */
        for (size_t qt = 0; qt < nb; qt++) {
            const uint32_t* picks = selected + qt * topk;
            for (size_t qslot = qt * TE; qslot < qt * TE + block_sizes[qt]; qslot++) {
                const size_t qtok = (size_t)slot_src[qslot];
                const float* qr = q + base + qtok * dim;
                float m = NEG_INF;
                double z = 0.0;
                for (size_t d = 0; d < dim; d++) acc[d] = 0.0;
                for (size_t pi = 0; pi < topk; pi++) {
                    const size_t kt = picks[pi];
                    for (size_t kslot = kt * TE; kslot < kt * TE + block_sizes[kt]; kslot++) {
                        const size_t ktok = (size_t)slot_src[kslot];
                        double dot = -0.0;
                        for (size_t d = 0; d < dim; d++)
                            dot += (double)qr[d] * (double)k[base + ktok * dim + d];
                        const float s = (float)(dot * (double)scale);
                        if (s > m) {
                            const double shrink = isfinite(m) ? exp((double)(m - s)) : 0.0;
                            z *= shrink;
                            for (size_t d = 0; d < dim; d++) acc[d] *= shrink;
                            m = s;
                        }
                        const double e = exp((double)(s - m));
                        z += e;
                        for (size_t d = 0; d < dim; d++)
                            acc[d] += e * (double)v[base + ktok * dim + d];
                    }
                }
                const size_t dst = base + qtok * dim;
                for (size_t d = 0; d < dim; d++) {
                    const float sparse = z > 0.0 ? (float)(acc[d] / z) : 0.0f;
                    const float c = coarse[qt * dim + d] * (gate ? gate[dst + d] : 1.0f);
                    out[dst + d] = c + sparse;
                }
            }
        }
    }
    free(qc);
    free(kc);
    free(vc);
    free(coarse);
    free(scores);
    free(exps);
    free(selected);
    free(acc);
    return 0;
}

/* ---- sequence-parallel helper ---------------------------------------------------- */

/* C/rt/sp.rs:16-28 */
void fvo_shard_ranges(size_t seq, size_t world, size_t* out) {
    if (world < 1) world = 1;
    const size_t base = seq / world, rem = seq % world;
    size_t start = 0;
    for (size_t r = 0; r < world; r++) {
        const size_t len = base + (r < rem ? 1 : 0);
        out[2 * r] = start;
        out[2 * r + 1] = len;
        start += len;
    }
}

/* ---- producer / consumer either side of the SDPA call --------------------------- */

/* C/rt/ops.rs:2304-2350 */
void fvo_qk_norm_rope_bhsd(const float* src, const float* w, const float* cos_t, const float* sin_t,
                           float* out, size_t batch, size_t seq, size_t heads, size_t d,
                           size_t src_width, size_t col_off, float eps) {
    const size_t width = heads * d;
    for (size_t b = 0; b < batch; b++)
        for (size_t s = 0; s < seq; s++) {
            const float* x = src + (b * seq + s) * src_width + col_off;
            float ss = 0.0f;
            for (size_t j = 0; j < width; j++) ss += x[j] * x[j];
            const float ms = ss / (float)width;
            const float inv = 1.0f / sqrtf(ms + eps);
            for (size_t h = 0; h < heads; h++) {
                float* o = out + ((b * heads + h) * seq + s) * d;
                for (size_t p = 0; p < d; p++) {
                    const size_t j = h * d + p;
                    if (!cos_t || !sin_t) {
                        o[p] = x[j] * inv * w[j];
                    } else {
                        const size_t even = p - (p & 1);
                        const size_t j0 = h * d + even;
                        const float x1 = x[j0] * inv * w[j0];
                        const float x2 = x[j0 + 1] * inv * w[j0 + 1];
                        const float c = cos_t[s * d + even];
                        const float sn = sin_t[s * d + even + 1];
                        o[p] = (p & 1) ? (x1 * sn + x2 * c) : (x1 * c - x2 * sn);
                    }
                }
            }
        }
}

/* C/wan/fuse.rs:321-342; C/rt/fuse/host.rs:93-96 (rms_factor), 217-241 (qk_norm),
 * 247-276 (qk_rope_head, interleaved pairing) */
void fvo_wan_qk_norm_rope16(const float* src, const float* w, const float* cos_t, const float* sin_t,
                            float* out, size_t batch, size_t seq, size_t heads, size_t d,
                            size_t src_width, size_t col_off, float eps) {
    const size_t width = heads * d;
    float* n = (float*)malloc(width * sizeof(float));
    for (size_t b = 0; b < batch; b++)
        for (size_t s = 0; s < seq; s++) {
            const float* x = src + (b * seq + s) * src_width + col_off;
            float ss = 0.0f;
            for (size_t j = 0; j < width; j++) ss += x[j] * x[j];
            const float inv = 1.0f / sqrtf(ss / (float)width + eps);
            for (size_t j = 0; j < width; j++) {
                const float t = fvo_bf16_round(x[j] * inv);
                n[j] = fvo_bf16_round(t * w[j]);
            }
            for (size_t h = 0; h < heads; h++) {
                float* o = out + ((b * heads + h) * seq + s) * d;
                const float* nh = n + h * d;
                for (size_t p = 0; p < d; p++) {
                    if (!cos_t || !sin_t) {
                        o[p] = nh[p];   /* already rounded (round_weighted) */
                    } else {
                        const size_t even = p - (p & 1);
                        const float x1 = nh[even], x2 = nh[even + 1];
                        const float cv = cos_t[s * d + even], sv = sin_t[s * d + even + 1];
                        o[p] = fvo_bf16_round((p & 1) ? (x2 * cv + x1 * sv) : (x1 * cv - x2 * sv));
                    }
                }
            }
        }
    free(n);
}

/* C/rt/ops.rs:2352-2372 */
void fvo_split_heads_bhsd(const float* src, float* out, size_t batch, size_t seq, size_t heads,
                          size_t d, size_t src_width, size_t col_off) {
    for (size_t b = 0; b < batch; b++)
        for (size_t h = 0; h < heads; h++)
            for (size_t s = 0; s < seq; s++)
                memcpy(out + ((b * heads + h) * seq + s) * d,
                       src + (b * seq + s) * src_width + col_off + h * d, d * sizeof(float));
}

/* C/rt/ops.rs:2374-2386 */
void fvo_merge_heads(const float* src, float* out, size_t batch, size_t heads, size_t seq, size_t d) {
    const size_t hd = heads * d;
    for (size_t b = 0; b < batch; b++)
        for (size_t s = 0; s < seq; s++)
            for (size_t h = 0; h < heads; h++)
                memcpy(out + (b * seq + s) * hd + h * d, src + ((b * heads + h) * seq + s) * d,
                       d * sizeof(float));
}

/* ---- VDN-H3 window mask --------------------------------------------------------------- */

/* C/rt/attn.rs:487-495 `bound` */
static long long vdn_bound(long long f, long long c, long long r, int hi) {
    if (c > 0) return hi ? (f / c + r + 1) * c - 1 : (f / c - r) * c;
    return hi ? f + r : f - r;
}

/* C/rt/attn.rs:497-510 */
int fvo_vdn_window_allows(size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                          size_t radius, size_t q, size_t k) {
    const size_t vs = video_start, ve = video_start + frames * frame_tokens;
    const size_t t = frame_tokens > 1 ? frame_tokens : 1;
    if (!(q >= vs && q < ve) || !(k >= vs && k < ve)) return 1;
    const size_t last = frames - 1;
    const size_t qf = (q - vs) / t, kf = (k - vs) / t;
    if (qf == 0 || kf == 0 || qf == last || kf == last) return 1;
    const long long kk = (long long)kf;
    return kk >= vdn_bound((long long)qf, (long long)chunk, (long long)radius, 0) &&
           kk <= vdn_bound((long long)qf, (long long)chunk, (long long)radius, 1);
}

/* C/rt/attn.rs:513-523 */
void fvo_vdn_window_dense_mask(size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                               size_t radius, size_t sq, size_t sk, float* mask) {
    for (size_t q = 0; q < sq; q++)
        for (size_t k = 0; k < sk; k++)
            mask[q * sk + k] =
                fvo_vdn_window_allows(video_start, frame_tokens, frames, chunk, radius, q, k) ? 0.0f : -1e9f;
}
