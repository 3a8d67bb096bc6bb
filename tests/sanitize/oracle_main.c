/* AddressSanitizer / UndefinedBehaviorSanitizer run of the CPU oracle (oracle/l2c.c, included as source): every
 * operator and a small model of each tensor-type mix in every arithmetic mode, on seeded data.  The numbers are not
 * checked here (tests/test_oracle.py does that); what counts is that the sanitizers stay silent.  Built and run by
 * tests/test_sanitizers.py. */
#include "../../oracle/l2c.c"

#include <stdio.h>

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(void) {
    rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
    return (uint32_t)(rng_state >> 33);
}
static float rndf(void) { return ((float)(rnd() & 0xFFFFFF) / 8388608.0f - 1.0f); }

/* random super-blocks with small finite fp16 scales */
static void *rand_blocks(int type, int64_t nb) {
    const int64_t bb = l2c_block_bytes(type);
    uint8_t *p = (uint8_t *)malloc((size_t)(nb * bb));
    for (int64_t i = 0; i < nb * bb; i++) p[i] = (uint8_t)rnd();
    for (int64_t b = 0; b < nb; b++) {
        const uint16_t d = l2c_fp32_to_fp16(0.01f * rndf()), dm = l2c_fp32_to_fp16(0.01f * rndf());
        uint8_t *q = p + b * bb;
        if (type == L2C_Q6_K) {
            memcpy(q + 208, &d, 2);
        } else {
            memcpy(q, &d, 2);
            memcpy(q + 2, &dm, 2);
        }
    }
    return p;
}
static void *rand_matrix(int type, int64_t ne0, int64_t ne1) {
    if (type == L2C_F32) {
        float *p = (float *)malloc((size_t)(ne0 * ne1) * 4);
        for (int64_t i = 0; i < ne0 * ne1; i++) p[i] = 0.02f * rndf();
        return p;
    }
    return rand_blocks(type, ne0 / 256 * ne1);
}

static void run_model(int t_att, int t_up, int t_down, int t_out, int neox, int n_kv) {
    l2c_config c = {512, 768, 2, 8, n_kv, 300, 24, 10000.0f, neox};
    const int kv_dim = c.dim / c.n_heads * c.n_kv_heads;
    void *keep[64];
    int nk = 0;
    float *ones = (float *)malloc(c.dim * 4);
    for (int i = 0; i < c.dim; i++) ones[i] = 1.0f + 0.1f * rndf();
    keep[nk++] = ones;
    const int modes[] = {0, 1, 2, 3, 3 | L2C_KV16};
    l2c_model *m = l2c_model_create(&c, 3);
#define SET(role, layer, type, ne0, ne1)                              \
    do {                                                              \
        void *p_ = rand_matrix(type, ne0, ne1);                       \
        keep[nk++] = p_;                                              \
        l2c_model_set_tensor(m, role, layer, type, p_, ne0, ne1);     \
    } while (0)
    SET(L2C_TOK_EMB, 0, t_out == L2C_F32 ? L2C_F32 : L2C_Q4_K, c.dim, c.vocab_size);
    l2c_model_set_tensor(m, L2C_RMS_FINAL, 0, L2C_F32, ones, c.dim, 1);
    SET(L2C_OUTPUT, 0, t_out, c.dim, c.vocab_size);
    for (int l = 0; l < c.n_layers; l++) {
        l2c_model_set_tensor(m, L2C_RMS_ATT, l, L2C_F32, ones, c.dim, 1);
        l2c_model_set_tensor(m, L2C_RMS_FFN, l, L2C_F32, ones, c.dim, 1);
        SET(L2C_WQ, l, t_att, c.dim, c.dim);
        SET(L2C_WK, l, t_att, c.dim, kv_dim);
        SET(L2C_WV, l, t_att, c.dim, kv_dim);
        SET(L2C_WO, l, t_att, c.dim, c.dim);
        SET(L2C_W1, l, t_up, c.dim, c.hidden_dim);
        SET(L2C_W3, l, t_up, c.dim, c.hidden_dim);
        SET(L2C_W2, l, t_down, c.hidden_dim, c.dim);
    }
    int32_t prompt[4] = {1, 17, 299, 0}, out[8];
    float *logits = (float *)malloc(c.vocab_size * 4), *kv = (float *)malloc((size_t)2 * c.seq_len * kv_dim * 4);
    for (unsigned k = 0; k < sizeof modes / sizeof modes[0]; k++) {
        l2c_state_reset(m);
        if (l2c_generate_greedy(m, prompt, 4, 0, 8, modes[k], out, logits) != 8) abort();
        /* up to the last position of the cache, then the cache read and written back whole */
        if (l2c_forward(m, out[7], c.seq_len - 1, modes[k], logits) != 0) abort();
        if (l2c_kv_read(m, 1, 0, c.seq_len, kv, kv + (size_t)c.seq_len * kv_dim) != 0) abort();
        if (l2c_kv_write(m, 0, 0, c.seq_len, kv, kv + (size_t)c.seq_len * kv_dim) != 0) abort();
        if (l2c_argmax(logits, c.vocab_size) < 0) abort();
    }
    free(logits);
    free(kv);
    l2c_model_destroy(m);
    for (int i = 0; i < nk; i++) free(keep[i]);
}

int main(void) {
    /* codecs and dot products: every type, several block counts */
    const int types[3] = {L2C_Q4_K, L2C_Q5_K, L2C_Q6_K};
    for (int ti = 0; ti < 3; ti++) {
        for (int64_t nb = 1; nb <= 17; nb += 8) {
            void *blk = rand_blocks(types[ti], nb);
            float *y = (float *)malloc((size_t)nb * 256 * 4), *x = (float *)malloc((size_t)nb * 256 * 4);
            for (int64_t i = 0; i < nb * 256; i++) x[i] = rndf();
            if (l2c_dequantize(types[ti], blk, nb, y) != 0) abort();
            void *q8 = malloc((size_t)nb * 292);
            l2c_quantize_q8_K(x, nb * 256, q8);
            int32_t *isc = (int32_t *)malloc((size_t)nb * 4), *imin = (int32_t *)malloc((size_t)nb * 4);
            for (int canon = 0; canon < 2; canon++) {
                (void)l2c_vecdot_f32act(types[ti], blk, nb, x, canon);
                (void)l2c_vecdot_q8k(types[ti], blk, q8, nb, canon, isc, imin);
            }
            free(isc), free(imin), free(q8), free(x), free(y), free(blk);
        }
    }
    /* the q8_K rule's corner cases: zero block, ties, huge and denormal values */
    {
        float x[1024];
        for (int i = 0; i < 1024; i++) x[i] = i < 256 ? 0.0f : (i < 512 ? (i & 1 ? 3.0f : -3.0f) : (i < 768 ? 1e30f * rndf() : 1e-40f * (float)i));
        uint8_t q8[4 * 292];
        l2c_quantize_q8_K(x, 1024, q8);
    }
    run_model(L2C_Q4_K, L2C_Q4_K, L2C_Q4_K, L2C_Q6_K, 0, 2);  /* Q4_K_S-like, grouped heads */
    run_model(L2C_Q5_K, L2C_Q5_K, L2C_Q6_K, L2C_Q6_K, 0, 4);  /* Q5_K_M-like */
    run_model(L2C_Q4_K, L2C_Q4_K, L2C_Q4_K, L2C_Q4_K, 1, 8);  /* Phi-3-like: neox, no grouping */
    run_model(L2C_F32, L2C_F32, L2C_F32, L2C_F32, 0, 8);      /* llama2.c-like */
    puts("oracle: sanitizers silent");
    return 0;
}
