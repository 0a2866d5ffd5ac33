/*
 * asan_check.c -- drives every entry point of the CPU oracle (rllama_oracle.c) on small, awkward sizes: row counts that are
 * not multiples of the 4-row tile, K extents that are not multiples of the 8 lanes, a one-position cache, the ends of the
 * cache, both modes, both probes.  TEST INFRASTRUCTURE ONLY.  `make -C oracle asan` builds it together with the oracle
 * under AddressSanitizer and UndefinedBehaviorSanitizer; tests/test_sanitizers.py runs it.  It checks nothing numerically
 * (tests/test_oracle.py does): it exists so that an out-of-bounds access or undefined behaviour in the oracle cannot hide.
 */
#include "rllama_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>

static uint32_t rng_state = 12345u;
static float frand(void) {
    rng_state = rng_state * 1664525u + 1013904223u;
    return ((float)(rng_state >> 8) / 16777216.0f - 0.5f) * 0.4f;
}

static void fill_f32(float *p, size_t n) {
    for (size_t i = 0; i < n; i++) p[i] = frand();
}

static void products(void) {
    const int ks[] = {1, 7, 8, 9, 15, 16, 17, 100};
    const int ns[] = {1, 3, 4, 5, 9};
    for (unsigned a = 0; a < sizeof ks / sizeof *ks; a++)
        for (unsigned b = 0; b < sizeof ns / sizeof *ns; b++)
            for (int rows = 1; rows <= 3; rows++) {
                const int k = ks[a], nw = ns[b];
                float *x = malloc(sizeof(float) * (size_t)rows * k), *w = malloc(sizeof(float) * (size_t)nw * k), *o = malloc(sizeof(float) * (size_t)rows * nw);
                uint16_t *xh = malloc(2 * (size_t)rows * k), *wh = malloc(2 * (size_t)nw * k), *oh = malloc(2 * (size_t)rows * nw);
                fill_f32(x, (size_t)rows * k);
                fill_f32(w, (size_t)nw * k);
                orc_f32_to_f16_array(x, xh, (size_t)rows * k);
                orc_f32_to_f16_array(w, wh, (size_t)nw * k);
                orc_matmul_transposed_f32(x, rows, w, nw, k, o);
                orc_matmul_transposed_f16(xh, rows, wh, nw, k, oh);
                orc_f16_to_f32_array(oh, o, (size_t)rows * nw);
                (void)orc_dot8_f32(x, w, k);
                (void)orc_dot8_f32_scalar(x, w, k);
                (void)orc_dot8_f16(xh, wh, k);
                float *bm = malloc(sizeof(float) * (size_t)k * nw), *sq = malloc(sizeof(float) * (size_t)rows * nw), *vv = malloc(sizeof(float) * (size_t)nw);
                fill_f32(bm, (size_t)k * nw);
                orc_matmul_f32_seqk(x, rows, bm, nw, k, sq);
                orc_vector_matrix_mul_f32(x, bm, k, nw, vv);
                free(x); free(w); free(o); free(xh); free(wh); free(oh); free(bm); free(sq); free(vv);
            }
}

static void rows_and_sampler(void) {
    for (int d = 1; d <= 33; d += 8) {
        float *x = malloc(sizeof(float) * (size_t)d), *w = malloc(sizeof(float) * (size_t)d), *o = malloc(sizeof(float) * (size_t)d);
        fill_f32(x, (size_t)d);
        fill_f32(w, (size_t)d);
        orc_rmsnorm_row(x, w, d, 1e-6, o);
        orc_softmax_row(x, d, o);
        free(x); free(w); free(o);
    }
    double fc[16 * 4 * 2];
    orc_freqs_cis(8, 16, 10000.0, fc);
    float q[2 * 8];
    fill_f32(q, 16);
    orc_rope_row(q, 2, 8, fc + 15 * 4 * 2);
    (void)orc_silu(0.3f);
    (void)orc_hsum8(q);
    for (uint32_t h = 0; h < 65536u; h += 257u) (void)orc_f32_to_f16_bits(orc_f16_bits_to_f32((uint16_t)h));
    (void)orc_f32_to_f16_hw(orc_f16_to_f32_hw(0x3c00));
    const int V = 37;
    float logits[37];
    fill_f32(logits, V);
    logits[5] = 200.0f; /* overflows the un-shifted softmax */
    int32_t ids[37], existing[3] = {0, 5, 0}, ties = 0;
    float probs[37], total = 0.0f, pr = 0.0f;
    for (int top_k = 1; top_k <= 40; top_k += 13) {
        const int n = orc_sample_candidates(logits, V, 0.7f, 0.9f, top_k, 0.8f, existing, 3, ids, probs, &total);
        (void)orc_sample_pick(ids, probs, n, total, 0.5f, &pr);
    }
    logits[5] = 1.0f;
    const int n = orc_sample_candidates(logits, V, 0.0f, 1.0f, V, 1.0f, NULL, 0, ids, probs, &total);
    (void)orc_sample_pick(ids, probs, n, total, 1.0f, &pr);
    (void)orc_sample_greedy(logits, V, 1.0f, &pr, &ties);
    logits[0] = NAN;
    (void)orc_sample_greedy(logits, V, 0.2f, NULL, NULL);
}

static void model(int force_f16, int dim, int heads, int ffn, int vocab, int max_seq) {
    orc_params p = {dim, 2, heads, ffn, vocab, max_seq, 1e-6, force_f16};
    orc_model *m = orc_model_create(&p);
    if (!m) exit(3);
    const size_t big = (size_t)(vocab > ffn ? vocab : ffn) * (size_t)dim;
    float *buf = malloc(sizeof(float) * big);
    uint16_t *bh = malloc(2 * big);
    struct { int kind, rows, cols; } t[] = {{ORC_WQ, dim, dim}, {ORC_WK, dim, dim}, {ORC_WV, dim, dim}, {ORC_WO, dim, dim}, {ORC_W1, ffn, dim},
                                            {ORC_W3, ffn, dim}, {ORC_W2, dim, ffn}, {ORC_ATTN_NORM, 1, dim}, {ORC_FFN_NORM, 1, dim}};
    for (int l = 0; l < 2; l++)
        for (unsigned i = 0; i < sizeof t / sizeof *t; i++) {
            fill_f32(buf, (size_t)t[i].rows * t[i].cols);
            if ((l + i) & 1) { /* both source dtypes */
                orc_f32_to_f16_array(buf, bh, (size_t)t[i].rows * t[i].cols);
                if (orc_model_set_tensor(m, t[i].kind, l, bh, t[i].rows, t[i].cols, ORC_F16)) exit(4);
            } else if (orc_model_set_tensor(m, t[i].kind, l, buf, t[i].rows, t[i].cols, ORC_F32)) exit(4);
        }
    fill_f32(buf, (size_t)vocab * dim);
    if (orc_model_set_tensor(m, ORC_TOK_EMB, 0, buf, vocab, dim, ORC_F32)) exit(4);
    fill_f32(buf, (size_t)vocab * dim);
    if (orc_model_set_tensor(m, ORC_OUTPUT, 0, buf, vocab, dim, ORC_F32)) exit(4);
    fill_f32(buf, (size_t)dim);
    if (orc_model_set_tensor(m, ORC_NORM, 0, buf, 1, dim, ORC_F32)) exit(4);
    if (!orc_model_set_tensor(m, ORC_WQ, 2, buf, dim, dim, ORC_F32)) exit(5);   /* layer out of range must be refused */
    if (!orc_model_set_tensor(m, ORC_WQ, 0, buf, dim + 1, dim, ORC_F32)) exit(5); /* wrong shape must be refused */

    float *logits = malloc(sizeof(float) * (size_t)vocab), *tap = malloc(sizeof(float) * 2 * (size_t)max_seq * dim);
    float *x = malloc(sizeof(float) * (size_t)max_seq * dim), *plane = malloc(sizeof(float) * (size_t)(dim / heads) * max_seq);
    int32_t *toks = malloc(sizeof(int32_t) * (size_t)max_seq);
    for (int i = 0; i < max_seq; i++) toks[i] = (i * 7 + 1) % vocab;
    for (int probe = 0; probe < 3; probe++) {
        orc_set_alt_order(probe == 1);
        orc_set_exact_sums(probe == 2);
        orc_caches *c = orc_caches_create(m);
        const int n_prompt = max_seq > 3 ? max_seq - 2 : 1;
        orc_set_layer_tap(tap);
        if (orc_forward(m, c, toks, n_prompt, 0, logits)) exit(6);
        orc_set_layer_tap(NULL);
        for (int pos = n_prompt; pos < max_seq; pos++)
            if (orc_forward(m, c, toks + pos, 1, pos, logits)) exit(6); /* up to the last position of the cache */
        if (!orc_forward(m, c, toks, 1, max_seq, logits)) exit(7);      /* past the end must be refused */
        if (!orc_forward(m, c, toks, 2, 1, logits)) exit(7);            /* n > 1 at start_pos > 0 must be refused */
        int32_t bad = vocab;
        if (!orc_forward(m, c, &bad, 1, 0, logits)) exit(7);            /* token id out of range must be refused */
        orc_caches *c2 = orc_caches_true_clone(c);
        orc_caches_shift_left(c2, 1);
        orc_caches_shift_left(c2, max_seq + 3); /* more shifts than columns */
        orc_caches_read(c2, 1, heads - 1, 1, plane);
        if (orc_embed(m, toks, n_prompt, x)) exit(8);
        orc_caches *c3 = orc_caches_create(m);
        if (orc_forward_layers(m, c3, x, n_prompt, 0, 0, 0, x)) exit(8);
        if (orc_forward_layers(m, c3, x, n_prompt, 0, 1, 1, x)) exit(8);
        if (!orc_forward_layers(m, c3, x, n_prompt, 0, 1, 2, x)) exit(9);
        if (orc_head(m, x, n_prompt, logits)) exit(8);
        orc_caches_free(c);
        orc_caches_free(c2);
        orc_caches_free(c3);
    }
    orc_set_alt_order(0);
    orc_set_exact_sums(0);
    free(logits); free(tap); free(x); free(plane); free(toks); free(buf); free(bh);
    orc_model_free(m);
}

int main(void) {
    for (int threads = 1; threads <= 3; threads += 2) {
        orc_set_threads(threads);
        orc_set_reference_threading(threads == 1);
        products();
        rows_and_sampler();
        for (int f16 = 0; f16 <= 1; f16++) {
            model(f16, 16, 2, 24, 11, 1);   /* a one-position cache */
            model(f16, 24, 3, 40, 13, 7);   /* head_dim 8, ffn and vocabulary no multiples of 4 x 8 */
            model(f16, 20, 2, 36, 9, 10);   /* head_dim 10: K extents that are no multiple of the 8 lanes */
        }
    }
    (void)orc_get_threads();
    printf("oracle: every entry point ran under the sanitizers\n");
    return 0;
}
