/*
 * abi_layer_ops.c — the layer ops and the runtime, driven from plain C the way
 * the reference's C engine and its own test programs drive a backend: link the
 * library, call the device.h-level symbols, compare against the CPU kernels.
 *
 * Modelled on the reference's device tests: inputs from the inline LCG they
 * use (tests/test_decode_position.c:30-34), one check() line per assertion,
 * non-zero exit on failure, "SKIP" when no device is present
 * (tests/test_device_memory.c:216-223). Cases:
 *   - vv_pos_add_dev / vv_dev_memcpy_d2d_at           (test_decode_position.c:70-112)
 *   - RoPE at a position only the device knows        (test_decode_position.c:220-238)
 *   - vv_rmsnorm_dev / vv_swiglu_dev at K in {1536, 3584, 8960, 18944},
 *     M in {1, 7, 285}                                 (test_int8_linear.c:295-354 shapes)
 *   - embedding gather, bit-exact
 *   - capture once, replay many                        (test_device_memory.c:164-212)
 *   - a linear layer (GEMM + bias, one row and a chunk), the multi-projection small-M form,
 *     causal attention (prefill, then a decode row on the same cache) and the greedy head
 * The CPU side is the oracle library (test infrastructure, never shipped).
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "vibevoice_hip.h"
#include "vv_oracle.h"

static uint32_t rng_state = 0xB5297A4Du;
static float frand(void) {
    rng_state = rng_state * 1664525u + 1013904223u;
    return ((float)(rng_state >> 8) / 8388608.0f) - 1.0f;
}

static int failures = 0;
static void check(int ok, const char* what) {
    printf("  %s %s\n", ok ? "ok  " : "FAIL", what);
    if (!ok) failures++;
}

/* max|got-ref| / max|ref|, the reference's tolerance scale (test_cpu_kernels.c:36-54) */
static double scaled_err(const uint16_t* got, const float* ref, size_t n) {
    double max_abs = 0.0, mag = 0.0;
    for (size_t i = 0; i < n; i++) {
        const double d = fabs((double)vvo_half_to_float(got[i]) - (double)ref[i]);
        if (d > max_abs) max_abs = d;
        if (fabs((double)ref[i]) > mag) mag = fabs((double)ref[i]);
    }
    return max_abs / (mag + 1e-9);
}

static void* to_dev(const void* h, size_t n) {
    void* d = NULL;
    if (vv_dev_alloc(&d, n ? n : 16) != VV_OK) return NULL;
    if (n && h) vv_dev_memcpy_h2d(d, h, n, NULL);
    return d;
}

static int* dev_int(int v) { return (int*)to_dev(&v, sizeof v); }

static int read_dev_int(const int* p) {
    int v = -1;
    vv_dev_stream_sync(NULL);
    vv_dev_memcpy_d2h(&v, p, sizeof v, NULL);
    return v;
}

static void test_position_plumbing(void) {
    printf("device-side position and index\n");
    int* a = dev_int(41);
    int* b = dev_int(0);
    check(vv_pos_add_dev(b, a, 1, NULL) == VV_OK && read_dev_int(b) == 42, "pos_add writes src + delta");
    check(vv_pos_add_dev(a, a, 1, NULL) == VV_OK && read_dev_int(a) == 42, "pos_add in place");

    enum { ROW = 512, AT = 7 };
    uint8_t pattern[ROW], got[ROW * 16];
    for (int i = 0; i < ROW; i++) pattern[i] = (uint8_t)(i * 7 + 3);
    void* base = to_dev(NULL, ROW * 16);
    void* src = to_dev(pattern, ROW);
    vv_dev_memset(base, 0, ROW * 16);
    int* idx = dev_int(AT);
    check(vv_dev_memcpy_d2d_at(base, src, ROW, idx, NULL) == VV_OK, "memcpy_d2d_at returns ok");
    vv_dev_stream_sync(NULL);
    vv_dev_memcpy_d2h(got, base, sizeof got, NULL);
    int clean = 1;
    for (int i = 0; i < ROW * 16; i++)
        if ((i < AT * ROW || i >= (AT + 1) * ROW) && got[i] != 0) clean = 0;
    check(memcmp(got + AT * ROW, pattern, ROW) == 0, "memcpy_d2d_at lands at (*d_index) * size");
    check(clean, "memcpy_d2d_at touches nothing else");
    vv_dev_free(a); vv_dev_free(b); vv_dev_free(base); vv_dev_free(src); vv_dev_free(idx);
}

static void test_rope_device_position(void) {
    printf("rope: host position == device position, and both == CPU kernel\n");
    enum { NQ = 28, NK = 4, HD = 128 };
    const size_t nq = (size_t)NQ * HD, nk = (size_t)NK * HD;
    uint16_t hq[NQ * HD], hk[NK * HD], ga[NQ * HD], gb[NQ * HD], gk[NK * HD];
    float ref[NQ * HD];
    for (size_t i = 0; i < nq; i++) hq[i] = vvo_float_to_half_rne(frand());
    for (size_t i = 0; i < nk; i++) hk[i] = vvo_float_to_half_rne(frand());
    void* xa = to_dev(hq, nq * 2);
    void* xb = to_dev(hq, nq * 2);
    int* d_p = dev_int(913);
    check(vv_rope_dev(xa, 1, NQ, HD, 913, NULL, 1000000.0f, NULL) == VV_OK, "rope (scalar position)");
    check(vv_rope_dev(xb, 1, NQ, HD, 0, d_p, 1000000.0f, NULL) == VV_OK, "rope (device position)");
    vv_dev_stream_sync(NULL);
    vv_dev_memcpy_d2h(ga, xa, nq * 2, NULL);
    vv_dev_memcpy_d2h(gb, xb, nq * 2, NULL);
    check(memcmp(ga, gb, nq * 2) == 0, "device position matches host position exactly");
    check(memcmp(ga, hq, nq * 2) != 0, "rope actually rotated something");
    vvo_rope_f16(hq, ref, NULL, 1, NQ, HD, 913, 1000000.0f);
    check(scaled_err(ga, ref, nq) <= 2e-3, "rope vs CPU kernel within 2e-3");

    /* Q and K in one launch == two launches */
    void* q2 = to_dev(hq, nq * 2);
    void* k1 = to_dev(hk, nk * 2);
    void* k2 = to_dev(hk, nk * 2);
    vv_rope_dev(k1, 1, NK, HD, 913, NULL, 1000000.0f, NULL);
    check(vv_rope_qk_dev(q2, k2, 1, NQ, NK, HD, 913, NULL, 1000000.0f, NULL) == VV_OK, "rope_qk");
    vv_dev_stream_sync(NULL);
    vv_dev_memcpy_d2h(gb, q2, nq * 2, NULL);
    check(memcmp(ga, gb, nq * 2) == 0, "rope_qk Q == rope Q");
    vv_dev_memcpy_d2h(gk, k1, nk * 2, NULL);
    vv_dev_memcpy_d2h(hk, k2, nk * 2, NULL);
    check(memcmp(gk, hk, nk * 2) == 0, "rope_qk K == rope K");
    vv_dev_free(xa); vv_dev_free(xb); vv_dev_free(d_p); vv_dev_free(q2); vv_dev_free(k1); vv_dev_free(k2);
}

static void test_norm_and_swiglu_shapes(void* st) {
    printf("rmsnorm / swiglu / add+rmsnorm vs CPU kernels\n");
    const int Ks[] = { 1536, 3584, 8960, 18944 };
    const int Ms[] = { 1, 7, 285 };
    for (int ki = 0; ki < 4; ki++) for (int mi = 0; mi < 3; mi++) {
        const int K = Ks[ki], M = Ms[mi];
        const size_t n = (size_t)M * K;
        uint16_t* h = malloc(n * 2);
        uint16_t* h2 = malloc(n * 2);
        uint16_t* hw = malloc((size_t)K * 2);
        uint16_t* got = malloc(n * 2);
        uint16_t* res = malloc(n * 2);
        float* ref = malloc(n * 4);
        for (size_t i = 0; i < n; i++) h[i] = vvo_float_to_half_rne(frand() * 4.0f);
        for (size_t i = 0; i < n; i++) h2[i] = vvo_float_to_half_rne(frand() * 3.0f);
        for (int i = 0; i < K; i++) hw[i] = vvo_float_to_half_rne(0.5f + frand() * 0.4f);
        void* dx = to_dev(h, n * 2);
        void* dx2 = to_dev(h2, n * 2);
        void* dw = to_dev(hw, (size_t)K * 2);
        void* dy = to_dev(NULL, n * 2);
        char what[96];

        vv_status_t s = vv_rmsnorm_dev(dx, dw, dy, M, K, 1e-6f, st);
        vv_dev_stream_sync(st);
        vv_dev_memcpy_d2h(got, dy, n * 2, NULL);
        vvo_rmsnorm_f16(h, hw, ref, NULL, M, K, 1e-6f);
        snprintf(what, sizeof what, "rmsnorm M=%d K=%d rel=%.2e", M, K, scaled_err(got, ref, n));
        check(s == VV_OK && scaled_err(got, ref, n) <= 2e-3, what);

        s = vv_swiglu_dev(dx, dx2, dy, (int)n, st);
        vv_dev_stream_sync(st);
        vv_dev_memcpy_d2h(got, dy, n * 2, NULL);
        vvo_swiglu_f16(h, h2, ref, NULL, n);
        snprintf(what, sizeof what, "swiglu  M=%d K=%d rel=%.2e", M, K, scaled_err(got, ref, n));
        check(s == VV_OK && scaled_err(got, ref, n) <= 2e-3, what);

        /* fused add+norm: residual bit-exact, normed within tolerance */
        memcpy(res, h, n * 2);
        vvo_add_rmsnorm_f16(res, h2, hw, ref, NULL, M, K, 1e-6f);
        s = vv_add_rmsnorm_dev(dx, dx2, dw, dy, M, K, 1e-6f, st);
        vv_dev_stream_sync(st);
        vv_dev_memcpy_d2h(got, dx, n * 2, NULL);
        const int exact = memcmp(got, res, n * 2) == 0;
        vv_dev_memcpy_d2h(got, dy, n * 2, NULL);
        snprintf(what, sizeof what, "add+norm M=%d K=%d residual exact, rel=%.2e", M, K,
                 scaled_err(got, ref, n));
        check(s == VV_OK && exact && scaled_err(got, ref, n) <= 2e-3, what);

        vv_dev_free(dx); vv_dev_free(dx2); vv_dev_free(dw); vv_dev_free(dy);
        free(h); free(h2); free(hw); free(got); free(res); free(ref);
    }
}

static void test_embedding(void* st) {
    printf("embedding gather\n");
    enum { V = 1000, H = 3584, T = 257 };
    uint16_t* table = malloc((size_t)V * H * 2);
    uint16_t* want = malloc((size_t)T * H * 2);
    uint16_t* got = malloc((size_t)T * H * 2);
    int32_t ids[T];
    for (size_t i = 0; i < (size_t)V * H; i++) { rng_state = rng_state * 1664525u + 1013904223u; table[i] = (uint16_t)(rng_state >> 12); }
    vvo_fill_ids(ids, T, 9, V);
    ids[0] = 0; ids[1] = V - 1; ids[2] = V - 1;
    vvo_embedding_f16(table, ids, want, T, H);
    void* dt = to_dev(table, (size_t)V * H * 2);
    void* di = to_dev(ids, sizeof ids);
    void* dout = to_dev(NULL, (size_t)T * H * 2);
    check(vv_embedding_dev(dt, (const int32_t*)di, dout, T, H, st) == VV_OK, "embedding returns ok");
    vv_dev_stream_sync(st);
    vv_dev_memcpy_d2h(got, dout, (size_t)T * H * 2, NULL);
    check(memcmp(got, want, (size_t)T * H * 2) == 0, "gather is bit-exact");
    vv_dev_free(dt); vv_dev_free(di); vv_dev_free(dout);
    free(table); free(want); free(got);
}

static void test_graph(void) {
    printf("graph: capture once, replay many\n");
    enum { RB = 32, NR = 16 };
    void *pos = to_dev(NULL, 4), *rows = to_dev(NULL, RB * NR), *row = to_dev(NULL, RB), *st = NULL;
    vv_dev_stream_create(&st);
    int zero = 0;
    uint8_t h[RB], back[RB * NR];
    static const uint8_t zeros[RB] = {0};
    for (int i = 0; i < RB; i++) h[i] = (uint8_t)(i + 1);
    vv_dev_memcpy_h2d(pos, &zero, 4, st);
    vv_dev_memset_async(rows, 0, RB * NR, st);
    vv_dev_memcpy_h2d(row, h, RB, st);
    vv_dev_stream_sync(st);
    void* g = NULL;
    check(vv_dev_graph_begin(st) == VV_OK, "begin");
    vv_dev_memcpy_d2d_at(rows, row, RB, (const int*)pos, st);
    vv_pos_add_dev((int*)pos, (const int*)pos, 1, st);
    check(vv_dev_graph_end(st, &g) == VV_OK && g, "end");
    int p = -1;
    vv_dev_memcpy_d2h(&p, pos, 4, st);
    vv_dev_stream_sync(st);
    check(p == 0, "capture ran nothing");
    for (int i = 0; i < 5; i++) check(vv_dev_graph_launch(g, st) == VV_OK, "launch");
    vv_dev_memcpy_d2h(&p, pos, 4, st);
    vv_dev_memcpy_d2h(back, rows, sizeof back, st);
    vv_dev_stream_sync(st);
    check(p == 5, "five replays advanced pos to 5");
    int bad = 0;
    for (int r = 0; r < NR; r++) bad |= memcmp(back + r * RB, r < 5 ? h : zeros, RB) != 0;
    check(!bad, "rows 0..4 written, the rest untouched");
    vv_dev_graph_destroy(g);

    check(vv_dev_graph_begin(st) == VV_OK, "begin 2");
    vv_dev_stream_sync(st);
    void* g2 = NULL;
    check(vv_dev_graph_end(st, &g2) != VV_OK && !g2, "a sync inside a capture breaks it");
    check(vv_pos_add_dev((int*)pos, (const int*)pos, 1, st) == VV_OK && read_dev_int(pos) == 6,
          "the stream still works after a broken capture");
    vv_dev_stream_destroy(st);
    vv_dev_free(pos); vv_dev_free(rows); vv_dev_free(row);
}

static uint16_t* rand_f16(size_t n, float scale) {
    uint16_t* h = (uint16_t*)malloc(n * 2);
    for (size_t i = 0; i < n; i++) h[i] = vvo_float_to_half_rne(scale * frand());
    return h;
}

static float* widen(const uint16_t* h, size_t n) {
    float* f = (float*)malloc(n * sizeof(float));
    for (size_t i = 0; i < n; i++) f[i] = vvo_half_to_float(h[i]);
    return f;
}

static void test_linear_attention_head(void* st) {
    printf("linear layers, attention, greedy head:\n");
    enum { K = 512, N = 384, NQ = 4, NKV = 2, HD = 128, T = 40, V = 1000 };
    uint16_t* w = rand_f16((size_t)N * K, 0.08f);
    uint16_t* bias = rand_f16(N, 0.3f);
    void *d_w = to_dev(w, (size_t)N * K * 2), *d_b = to_dev(bias, N * 2);
    const int rows[3] = {1, 29, 200};
    for (int c = 0; c < 3; c++) {
        const int M = rows[c];
        uint16_t* x = rand_f16((size_t)M * K, 1.0f);
        float* xf = widen(x, (size_t)M * K);
        float* ref = (float*)malloc((size_t)M * N * sizeof(float));
        vvo_gemm_f16w(xf, w, bias, ref, M, N, K);
        void *d_x = to_dev(x, (size_t)M * K * 2), *d_y = to_dev(NULL, (size_t)M * N * 2);
        vv_status_t s = vv_gemm_fp16_dev(d_x, d_w, d_y, M, N, K, 1.0f, 0.0f, st);
        if (s == VV_OK) s = vv_bias_add_dev(d_y, d_b, M, N, st);
        uint16_t* y = (uint16_t*)malloc((size_t)M * N * 2);
        vv_dev_memcpy_d2h(y, d_y, (size_t)M * N * 2, st);
        vv_dev_stream_sync(st);
        char what[96];
        snprintf(what, sizeof what, "GEMM + bias, M=%d: scaled error %.2e", M, scaled_err(y, ref, (size_t)M * N));
        check(s == VV_OK && scaled_err(y, ref, (size_t)M * N) <= 2e-3, what);
        if (M == 29) {      /* the reference's small-M entry point: one launch, the same bits */
            void* d_y2 = to_dev(NULL, (size_t)M * N * 2);
            vv_skinny_proj_t p = {d_w, NULL, d_b, d_y2, N};
            s = vv_skinny_linear_dev(d_x, 0, &p, 1, M, K, 1.0f, st);
            uint16_t* y2 = (uint16_t*)malloc((size_t)M * N * 2);
            vv_dev_memcpy_d2h(y2, d_y2, (size_t)M * N * 2, st);
            vv_dev_stream_sync(st);
            check(s == VV_OK && memcmp(y, y2, (size_t)M * N * 2) == 0, "vv_skinny_linear_dev == GEMM + bias add, bit for bit");
            free(y2); vv_dev_free(d_y2);
        }
        free(x); free(xf); free(ref); free(y); vv_dev_free(d_x); vv_dev_free(d_y);
    }

    /* attention: T rows over their own K/V, then one more row as a decode step on the same cache */
    uint16_t *q = rand_f16((size_t)(T + 1) * NQ * HD, 1.5f), *k = rand_f16((size_t)(T + 1) * NKV * HD, 1.0f),
             *v = rand_f16((size_t)(T + 1) * NKV * HD, 1.0f);
    float *qf = widen(q, (size_t)(T + 1) * NQ * HD), *kf = widen(k, (size_t)(T + 1) * NKV * HD),
          *vf = widen(v, (size_t)(T + 1) * NKV * HD);
    float* aref = (float*)malloc((size_t)(T + 1) * NQ * HD * sizeof(float));
    vvo_attention_prefill_f32(qf, kf, vf, aref, NQ, NKV, HD, T + 1, 0, T + 1, 1);
    void *d_q = to_dev(q, (size_t)(T + 1) * NQ * HD * 2), *d_k = to_dev(k, (size_t)(T + 1) * NKV * HD * 2),
         *d_v = to_dev(v, (size_t)(T + 1) * NKV * HD * 2), *d_o = to_dev(NULL, (size_t)(T + 1) * NQ * HD * 2);
    const vv_kv_view_t view = {d_k, d_v, NULL, NULL, NULL, 0, NKV, HD};
    const int backend = vv_attn_resolve(0, 0, false, NQ, NKV, HD);
    void* scratch = to_dev(NULL, vv_attn_scratch_bytes(NQ, NKV, HD));
    vv_status_t s = vv_attn_prefill(backend, d_q, &view, d_o, NQ, T, 0, T, true, scratch, st);
    if (s == VV_OK)
        s = vv_attn_decode(backend, (char*)d_q + (size_t)T * NQ * HD * 2, &view, (char*)d_o + (size_t)T * NQ * HD * 2,
                           NQ, T + 1, NULL, scratch, st);
    uint16_t* o = (uint16_t*)malloc((size_t)(T + 1) * NQ * HD * 2);
    vv_dev_memcpy_d2h(o, d_o, (size_t)(T + 1) * NQ * HD * 2, st);
    vv_dev_stream_sync(st);
    check(backend != 0 && s == VV_OK && scaled_err(o, aref, (size_t)T * NQ * HD) <= 2e-3, "causal prefill attention");
    check(scaled_err(o + (size_t)T * NQ * HD, aref + (size_t)T * NQ * HD, (size_t)NQ * HD) <= 2e-3,
          "decode attention on the same cache");

    /* greedy head: logits in FP32, the token the in-order scan picks from them */
    uint16_t *table = rand_f16((size_t)V * K, 0.05f), *h = rand_f16(K, 1.0f);
    void *d_t = to_dev(table, (size_t)V * K * 2), *d_h = to_dev(h, K * 2), *d_l = to_dev(NULL, V * 4),
         *d_sv = to_dev(NULL, 256 * 4), *d_si = to_dev(NULL, 256 * 4);
    int* d_tok = dev_int(-1);
    s = vv_lm_head_gemv_dev(d_h, d_t, d_l, V, K, st);
    if (s == VV_OK) s = vv_argmax_dev(d_l, V, d_sv, d_si, d_tok, NULL, st);
    float* logits = (float*)malloc(V * sizeof(float));
    vv_dev_memcpy_d2h(logits, d_l, V * 4, st);
    vv_dev_stream_sync(st);
    int32_t want = -2;
    vvo_argmax_first(logits, V, &want, NULL);
    check(s == VV_OK && read_dev_int(d_tok) == want, "LM head + on-device argmax");

    free(w); free(bias); free(q); free(k); free(v); free(qf); free(kf); free(vf); free(aref); free(o);
    free(table); free(h); free(logits);
    void* frees[] = {d_w, d_b, d_q, d_k, d_v, d_o, scratch, d_t, d_h, d_l, d_sv, d_si, d_tok};
    for (size_t i = 0; i < sizeof frees / sizeof frees[0]; i++) vv_dev_free(frees[i]);
}

int main(void) {
    if (vv_dev_device_count() <= 0) {
        printf("SKIP: no device available\n");
        return 0;
    }
    char name[128] = "";
    size_t total = 0, freem = 0;
    int cus = 0;
    vv_dev_get_device_name(0, name, sizeof name);
    vv_dev_get_device_info(0, &total, &freem, &cus);
    printf("backend %s, device 0: %s, %.1f/%.1f GiB free, %d CUs\n", vv_dev_backend_name(), name,
           freem / 1073741824.0, total / 1073741824.0, cus);
    check(total > 0 && freem <= total && cus > 0, "device info");
    void* st = NULL;
    check(vv_dev_stream_create(&st) == VV_OK && st, "stream");

    test_position_plumbing();
    test_rope_device_position();
    test_norm_and_swiglu_shapes(st);
    test_embedding(st);
    test_graph();
    test_linear_attention_head(st);
    vv_dev_stream_destroy(st);

    if (failures) {
        printf("=== %d check(s) failed ===\n", failures);
        return 1;
    }
    printf("=== all C ABI checks passed ===\n");
    return 0;
}
