// Drives the oracle's C functions on odd small shapes; built with -fsanitize=address,undefined by
// tests/test_c_abi.py (an out-of-bounds access or undefined operation in the checker aborts the run).
#include <stdio.h>
#include <stdlib.h>
#include <stdint.h>
#include "fv_oracle.h"
static float* rnd(size_t n, unsigned seed) { float* p = malloc(n * sizeof(float)); for (size_t i = 0; i < n; i++) { seed = seed * 1664525u + 1013904223u; p[i] = ((seed >> 8) & 0xffff) / 32768.0f - 1.0f; } return p; }
int main(void) {
    for (int t = 0; t < 4; t++) {
        size_t bh = 3, sq = 5 + 7 * t, sk = 9 + 13 * t, d = 8 + 8 * t;
        float *q = rnd(bh * sq * d, 1), *k = rnd(bh * sk * d, 2), *v = rnd(bh * sk * d, 3), *o = malloc(bh * sq * d * 4);
        float* mask = rnd(sq * sk, 4);
        fvo_sdpa_composed(q, k, v, NULL, o, bh, sq, sk, d, 0.3f, 2);
        fvo_sdpa_composed(q, k, v, mask, o, bh, sq, sk, d, 0.3f, 1);
        int64_t rows[3] = {0, (int64_t)sq / 2, (int64_t)sq - 1}, bc[3] = {4, 2, 1};
        float* orow = malloc(bh * 3 * d * 4);
        fvo_sdpa_composed_rows(q, k, v, bc, rows, 3, orow, bh, sq, sk, d, 0.3f, 2);
        fvo_sdpa_composed_rows(q, k, v, NULL, rows, 3, orow, bh, sq, sk, d, 0.3f, 1);
        fvo_sdpa_f64(q, k, v, bc, o, bh, sq, sk, d, 0.3, 2);
        fvo_sdpa_f64_rows(q, k, v, NULL, rows, 3, orow, bh, sq, sk, d, 0.3, 2);
        fvo_softmax_last(mask, mask, sq, sk);
        float* m2 = malloc(sq * sk * 4);
        fvo_block_causal_dense_mask(4, 2, 1, sq, sk, m2);
        fvo_vdn_window_dense_mask(1, 3, 3, 2, 1, sq, sk, m2);
        free(q); free(k); free(v); free(o); free(mask); free(orow); free(m2);
    }
    size_t grids[3][3] = {{5, 6, 7}, {4, 4, 4}, {1, 9, 3}};
    for (int gi = 0; gi < 3; gi++) {
        size_t dims[5];
        fvo_tile_plan(grids[gi][0], grids[gi][1], grids[gi][2], dims, NULL, NULL, NULL);
        size_t nb = dims[0] * dims[1] * dims[2], seq = dims[3], padded = dims[4], dim = 16, b = 1, heads = 2;
        int32_t* slot_src = malloc(padded * 4); uint32_t *token_slot = malloc(seq * 4), *bs = malloc(nb * 4);
        fvo_tile_plan(grids[gi][0], grids[gi][1], grids[gi][2], dims, slot_src, token_slot, bs);
        float *q = rnd(heads * seq * dim, 5), *k = rnd(heads * seq * dim, 6), *v = rnd(heads * seq * dim, 7), *g = rnd(heads * seq * dim, 8);
        float* out = malloc(heads * seq * dim * 4);
        size_t topk = fvo_topk_for(0.5, nb);
        uint32_t* sel = malloc(heads * nb * topk * 4);
        fvo_vsa_attention_host(q, k, v, g, slot_src, bs, seq, nb, topk, b, heads, dim, 0.25f, out, sel);
        fvo_vsa_attention_host(q, k, v, NULL, slot_src, bs, seq, nb, nb, b, heads, dim, 0.25f, out, NULL);
        float *qc = malloc(heads * nb * dim * 4), *sc = malloc(heads * nb * nb * 4);
        fvo_vsa_tile_mean(q, slot_src, bs, qc, heads, seq, dim, nb, 0);
        fvo_vsa_tile_mean(q, slot_src, bs, qc, heads, seq, dim, nb, 1);
        fvo_vsa_coarse_scores(qc, qc, sc, heads, nb, dim, 0.25f);
        fvo_topk_device_order(sc, sel, heads * nb, nb, topk);
        fvo_topk_host_order(sc, sel, heads * nb, nb, topk);
        float* sparse = rnd(heads * nb * 64 * dim, 9);
        fvo_vsa_combine(sparse, qc, g, slot_src, out, heads, seq, dim, nb, 0, nb, 0);
        fvo_vsa_combine(sparse, qc, NULL, slot_src, out, heads, seq, dim, nb, 0, nb, 1);
        if (nb > 1) fvo_vsa_combine(sparse, qc, g, slot_src, out, heads, seq, dim, nb, 1, nb - 1, 1);
        free(slot_src); free(token_slot); free(bs); free(q); free(k); free(v); free(g); free(out); free(sel); free(qc); free(sc); free(sparse);
    }
    {
        size_t batch = 2, seq = 11, heads = 3, d = 8, width = 3 * heads * d;
        float *src = rnd(batch * seq * width, 10), *w = rnd(heads * d, 11), *c = rnd(seq * d, 12), *s = rnd(seq * d, 13);
        float *out = malloc(batch * heads * seq * d * 4), *back = malloc(batch * seq * heads * d * 4);
        fvo_qk_norm_rope_bhsd(src, w, c, s, out, batch, seq, heads, d, width, heads * d, 1e-6f);
        fvo_qk_norm_rope_bhsd(src, w, NULL, NULL, out, batch, seq, heads, d, width, 0, 1e-6f);
        fvo_wan_qk_norm_rope16(src, w, c, s, out, batch, seq, heads, d, width, heads * d, 1e-6f);
        fvo_split_heads_bhsd(src, out, batch, seq, heads, d, width, 2 * heads * d);
        fvo_merge_heads(out, back, batch, heads, seq, d);
        size_t sr[2 * 5]; fvo_shard_ranges(37, 5, sr);
        free(src); free(w); free(c); free(s); free(out); free(back);
    }
    puts("oracle sanitizer run: ok");
    return 0;
}
