/*
 * rustane_oracle.c -- CPU restatement of the rustane decode path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker the HIP decode backend is compared against.  Nothing in the
 * shipped library links, loads or calls it: only the tests, the smoke check and the CPU-baseline
 * leg of the benchmark do.
 *
 * The reference runs its "naive" path partly on the Apple Neural Engine (fp16 inside) and its
 * cached path in fp32 Metal shaders; neither can be built off macOS.  This file restates, in
 * plain fp32 C, the arithmetic those two paths define.  Every function cites the reference
 * lines it follows (paths relative to the reference root).
 *
 * Pinning status (which independent check covers each function; see tests/test_oracle_*.py):
 *   orc_rmsnorm*            reference known answers cpu/rmsnorm.rs:245-277 + closed form
 *   orc_embedding           reference known answer cpu/embedding.rs:51-62
 *   orc_rope_inplace        closed form, pos-0 identity, norm preservation, relative-position
 *   GEMV / GEMM helpers     fp64 brute force on tiny shapes, index conventions of
 *                           tests/phase4_pretraining_checks.rs:745-787
 *   attention               fp64 brute-force softmax, n=1 -> v0, uniform K -> mean V
 *   orc_decode_* (cached)   equals row t of orc_forward_window; collapses to
 *                           LMhead(RMSNorm(embed[tok])) when wo = w2 = 0 (the reference's own
 *                           test regime, layer.rs:706-709)
 *   heads (argmax/top-k/    integer-exact against a sort with (value desc, index asc); the
 *    merge/block stats)     log-sum-exp identity; materialised block == slice of full logits
 *   RNG / samplers          hand-computed LCG known answers; inverse-CDF brute force; the block draw
 *                           (orc_sample_block_from_stats) against its float64 definition on either side
 *                           of every threshold, with overflowing / underflowing maxima, dead blocks and
 *                           a short last block; block-then-token draws against softmax(logits / T)
 *   ANE fp16-internal numerics and MPS accumulation order: parity unpinned (not reachable
 *   off Apple hardware); this oracle is fp32, the precision of the reference's Metal path.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_RMS_EPS 1e-5f          /* cpu/rmsnorm.rs EPS, metal-decode/src/lib.rs:14 */
#define ORC_BLOCK 256              /* metal-decode/src/lib.rs:156 argmax_threads */
#define ORC_MAX_TOPK 32            /* metal-decode/src/lib.rs:15 */

typedef struct {
    int32_t dim, hidden, heads, kv_heads, hd, seq, nlayers, vocab, q_dim, kv_dim, gqa_ratio;
    int32_t ffn_activation;        /* 0 = SwiGLU, 1 = LeakyReluSq (model.rs:3-25) */
} orc_config;

typedef struct {
    const float *wq, *wk, *wv, *wo, *w1, *w3, *w2, *gamma1, *gamma2;   /* layer.rs:19-36 */
} orc_layer;

typedef struct orc_model {
    orc_config cfg;
    orc_layer *layers;
    const float *gamma_final, *embed;
    int kv_round_bf16;             /* round K (post-RoPE) and V to bf16 when they enter the cache */
    float alpha;                   /* 1/sqrt(2L): layer.rs:1300, metal-decode/src/lib.rs:201 */
    float *rope_cos, *rope_sin;    /* [seq][hd/2] */
    float **kc, **vc;              /* per layer [seq][kv_dim] row-major: lib.rs:1049-1050 */
    int len;
    float *xf_last;                /* final-normed state of the last cached step (lib.rs:997) */
} orc_model;

/* ------------------------------------------------------------------ helpers */

static float bf16_round(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7f800000u) == 0x7f800000u) return f;          /* inf / nan unchanged */
    u += 0x7fffu + ((u >> 16) & 1u);                         /* round to nearest even */
    u &= 0xffff0000u;
    memcpy(&f, &u, 4);
    return f;
}

void orc_bf16_round_inplace(float *x, size_t n) {
    #pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) x[i] = bf16_round(x[i]);
}

/* cpu/rmsnorm.rs:149-183 with seq = 1 (decode.rs:101-108); metal-decode lib.rs:1354-1378 */
void orc_rmsnorm(const float *x, const float *gamma, float *out, int dim) {
    float ss = 0.0f;
    for (int d = 0; d < dim; ++d) ss += x[d] * x[d];
    float inv = 1.0f / sqrtf(ss * (1.0f / (float)dim) + ORC_RMS_EPS);
    for (int d = 0; d < dim; ++d) out[d] = x[d] * inv * gamma[d];
}

/* cpu/rmsnorm.rs:149-183, channel-first [dim, seq] */
void orc_rmsnorm_channel_first(const float *x, const float *gamma, float *out, float *rms_inv,
                               int dim, int seq) {
    for (int s = 0; s < seq; ++s) rms_inv[s] = 0.0f;
    for (int d = 0; d < dim; ++d)
        for (int s = 0; s < seq; ++s) rms_inv[s] += x[(size_t)d * seq + s] * x[(size_t)d * seq + s];
    float inv_dim = 1.0f / (float)dim;
    for (int s = 0; s < seq; ++s) rms_inv[s] = 1.0f / sqrtf(rms_inv[s] * inv_dim + ORC_RMS_EPS);
    for (int d = 0; d < dim; ++d)
        for (int s = 0; s < seq; ++s)
            out[(size_t)d * seq + s] = x[(size_t)d * seq + s] * rms_inv[s] * gamma[d];
}

/* cpu/embedding.rs:8-16: out[t, :] = embed[tokens[t], :] */
void orc_embedding(const float *embed, int dim, const uint32_t *tokens, int n, float *out) {
    for (int t = 0; t < n; ++t)
        memcpy(out + (size_t)t * dim, embed + (size_t)tokens[t] * dim, sizeof(float) * dim);
}

/* kernels/sdpa_fwd.rs:18-33 and metal-decode lib.rs:1392-1408:
 * theta = pos / 10000^(2i/hd), pairs (2i, 2i+1) inside each head. */
void orc_rope_table(int seq, int hd, float *cos_t, float *sin_t) {
    int pairs = hd / 2;
    for (int p = 0; p < seq; ++p)
        for (int i = 0; i < pairs; ++i) {
            float theta = (float)p / powf(10000.0f, 2.0f * (float)i / (float)hd);
            cos_t[(size_t)p * pairs + i] = cosf(theta);
            sin_t[(size_t)p * pairs + i] = sinf(theta);
        }
}

/* x holds n_heads*hd values; rotate every pair in place for position pos (lib.rs:1392-1408) */
void orc_rope_inplace(float *x, int n_heads, int hd, int pos) {
    int pairs = hd / 2;
    for (int h = 0; h < n_heads; ++h)
        for (int i = 0; i < pairs; ++i) {
            float theta = (float)pos / powf(10000.0f, 2.0f * (float)i / (float)hd);
            float c = cosf(theta), s = sinf(theta);
            float e = x[h * hd + 2 * i], o = x[h * hd + 2 * i + 1];
            x[h * hd + 2 * i] = e * c - o * s;
            x[h * hd + 2 * i + 1] = o * c + e * s;
        }
}

static void rope_rows(const orc_model *m, float *x, int n_heads, int pos) {
    int hd = m->cfg.hd, pairs = hd / 2;
    const float *ct = m->rope_cos + (size_t)pos * pairs, *st = m->rope_sin + (size_t)pos * pairs;
    for (int h = 0; h < n_heads; ++h)
        for (int i = 0; i < pairs; ++i) {
            float e = x[h * hd + 2 * i], o = x[h * hd + 2 * i + 1];
            x[h * hd + 2 * i] = e * ct[i] - o * st[i];
            x[h * hd + 2 * i + 1] = o * ct[i] + e * st[i];
        }
}

/* Y[t, o] = sum_d X[t, d] * W[d*O + o]   (weights with row = input channel: wq wk wv wo w1 w3;
 * lib.rs:533-556 transposeLeft GEMV, sdpa_fwd.rs:167, dyn_matmul.rs:420-431, ffn_fused.rs:114) */
void orc_gemm_in_major(const float *X, int T, int D, const float *W, int O, float *Y) {
    const int TB = 8, OB = 512;
    int n_tb = (T + TB - 1) / TB, n_ob = (O + OB - 1) / OB;
    #pragma omp parallel for collapse(2) schedule(dynamic)
    for (int tb = 0; tb < n_tb; ++tb)
        for (int ob = 0; ob < n_ob; ++ob) {
            int t0 = tb * TB, t1 = t0 + TB < T ? t0 + TB : T;
            int o0 = ob * OB, o1 = o0 + OB < O ? o0 + OB : O;
            float acc[8][512];
            for (int t = t0; t < t1; ++t)
                for (int o = o0; o < o1; ++o) acc[t - t0][o - o0] = 0.0f;
            for (int d = 0; d < D; ++d) {
                const float *w = W + (size_t)d * O;
                for (int t = t0; t < t1; ++t) {
                    float xv = X[(size_t)t * D + d];
                    float *a = acc[t - t0];
                    for (int o = o0; o < o1; ++o) a[o - o0] += xv * w[o];
                }
            }
            for (int t = t0; t < t1; ++t)
                for (int o = o0; o < o1; ++o) Y[(size_t)t * O + o] = acc[t - t0][o - o0];
        }
}

/* Y[t, o] = sum_k X[t, k] * W[o*K + k]   (weights with row = output channel: w2 and the tied
 * LM head; lib.rs:1189-1201, ffn_fused.rs:154-174, full_model.rs:419-428, lib.rs:1537-1540) */
void orc_gemm_out_major(const float *X, int T, int K, const float *W, int O, float *Y) {
    #pragma omp parallel for schedule(static)
    for (int o = 0; o < O; ++o) {
        const float *w = W + (size_t)o * K;
        for (int t = 0; t < T; ++t) {
            const float *x = X + (size_t)t * K;
            float acc = 0.0f;
            for (int k = 0; k < K; ++k) acc += x[k] * w[k];
            Y[(size_t)t * O + o] = acc;
        }
    }
}

static float gate_act(int act, float h1, float h3) {
    if (act == 1) {                                  /* ffn_fused.rs:145-148 leaky_relu(x,0.5)^2 */
        float l = h1 > 0.0f ? h1 : 0.5f * h1;
        return l * l * h3;
    }
    float sig = 1.0f / (1.0f + expf(-h1));           /* lib.rs:1510-1512, ffn_fused.rs:141-144 */
    return h1 * sig * h3;
}

/* softcap: decode.rs:120-124, full_model.rs:432-436, lib.rs:1663-1665 */
static float softcap_f(float x, float cap) { return cap > 0.0f ? cap * tanhf(x / cap) : x; }

/* One query row of causal attention for every head over cache rows [0, n)  (lib.rs:1426-1489;
 * sdpa_fwd.rs:325-354 masks t2 > t with -65504 before the softmax, which in fp32 is the same as
 * leaving those positions out). */
void orc_attend_row(const orc_config *c, const float *q, const float *kc, const float *vc,
                    int n, float *out, float *scores) {
    int hd = c->hd, KV = c->kv_dim;
    float scale = 1.0f / sqrtf((float)hd);
    for (int h = 0; h < c->heads; ++h) {
        int g = h / (c->gqa_ratio > 0 ? c->gqa_ratio : 1);
        const float *qh = q + h * hd;
        float mx = -3.402823466e+38f;
        for (int t = 0; t < n; ++t) {
            const float *k = kc + (size_t)t * KV + g * hd;
            float s = 0.0f;
            for (int j = 0; j < hd; ++j) s += qh[j] * k[j];
            s *= scale;
            scores[t] = s;
            if (s > mx) mx = s;
        }
        float sum = 0.0f;
        for (int t = 0; t < n; ++t) { scores[t] = expf(scores[t] - mx); sum += scores[t]; }
        float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
        float *o = out + h * hd;
        for (int j = 0; j < hd; ++j) o[j] = 0.0f;
        for (int t = 0; t < n; ++t) {
            float p = scores[t] * inv;
            const float *v = vc + (size_t)t * KV + g * hd;
            for (int j = 0; j < hd; ++j) o[j] += p * v[j];
        }
    }
}

/* ------------------------------------------------------------------ model */

orc_model *orc_create(const orc_config *cfg, const orc_layer *layers, const float *gamma_final,
                      const float *embed, int kv_round_bf16) {
    orc_model *m = (orc_model *)calloc(1, sizeof(orc_model));
    m->cfg = *cfg;
    m->layers = (orc_layer *)malloc(sizeof(orc_layer) * cfg->nlayers);
    memcpy(m->layers, layers, sizeof(orc_layer) * cfg->nlayers);
    m->gamma_final = gamma_final;
    m->embed = embed;
    m->kv_round_bf16 = kv_round_bf16;
    m->alpha = 1.0f / sqrtf(2.0f * (float)cfg->nlayers);
    m->rope_cos = (float *)malloc(sizeof(float) * cfg->seq * (cfg->hd / 2));
    m->rope_sin = (float *)malloc(sizeof(float) * cfg->seq * (cfg->hd / 2));
    orc_rope_table(cfg->seq, cfg->hd, m->rope_cos, m->rope_sin);
    m->kc = (float **)calloc(cfg->nlayers, sizeof(float *));
    m->vc = (float **)calloc(cfg->nlayers, sizeof(float *));
    for (int l = 0; l < cfg->nlayers; ++l) {
        m->kc[l] = (float *)calloc((size_t)cfg->seq * cfg->kv_dim, sizeof(float));
        m->vc[l] = (float *)calloc((size_t)cfg->seq * cfg->kv_dim, sizeof(float));
    }
    m->xf_last = (float *)calloc(cfg->dim, sizeof(float));
    m->len = 0;
    return m;
}

void orc_destroy(orc_model *m) {
    if (!m) return;
    for (int l = 0; l < m->cfg.nlayers; ++l) { free(m->kc[l]); free(m->vc[l]); }
    free(m->kc); free(m->vc); free(m->layers); free(m->rope_cos); free(m->rope_sin);
    free(m->xf_last); free(m);
}

int orc_len(const orc_model *m) { return m->len; }
/* lib.rs:213-215 */
void orc_set_len(orc_model *m, int len) { m->len = len < m->cfg.seq ? len : m->cfg.seq; }

/* lib.rs:217-237: cache[pos*KV + d] = k_rope_cf[d*S + pos] for pos < live_len, rest zero */
void orc_seed_layer_cache_from_channel_first(orc_model *m, int layer, int live_len,
                                             const float *k_rope_cf, const float *v_cf) {
    int S = m->cfg.seq, KV = m->cfg.kv_dim;
    if (live_len > S) live_len = S;
    memset(m->kc[layer], 0, sizeof(float) * (size_t)S * KV);
    memset(m->vc[layer], 0, sizeof(float) * (size_t)S * KV);
    for (int pos = 0; pos < live_len; ++pos)
        for (int d = 0; d < KV; ++d) {
            m->kc[layer][(size_t)pos * KV + d] = k_rope_cf[(size_t)d * S + pos];
            m->vc[layer][(size_t)pos * KV + d] = v_cf[(size_t)d * S + pos];
        }
}

const float *orc_kcache(const orc_model *m, int layer) { return m->kc[layer]; }
const float *orc_vcache(const orc_model *m, int layer) { return m->vc[layer]; }

/* Full-window forward: the arithmetic of full_model.rs:336-437 + layer.rs:1287-1431 +
 * kernels/{sdpa_fwd,dyn_matmul,ffn_fused}.rs for the first n_rows positions of the window
 * `input` (positions 0..n_rows-1, causal).  The reference always evaluates all cfg.seq rows of
 * a zero-padded window; causal masking makes rows < n_live independent of the padding, so
 * passing n_rows = n_live gives the same rows, and n_rows = cfg.seq restates the full cost.
 *   logits_out  [n_logit_rows][vocab] for the LAST n_logit_rows positions of the n_rows computed
 *   k_cf, v_cf  nullable, per layer channel-first [kv_dim][seq] (ForwardCache.k_rope / .v,
 *               layer.rs:52-67; the reference tiles KV heads to q_dim channels under GQA, this
 *               keeps kv_dim channels, which is what lib.rs:228-234 reads for MHA)
 * Also leaves the row-major K/V of these rows in the model's own cache and sets len = n_rows. */
int orc_forward_window(orc_model *m, const uint32_t *input, int n_rows, float softcap,
                       int n_logit_rows, float *logits_out, float *k_cf, float *v_cf) {
    const orc_config *c = &m->cfg;
    int D = c->dim, Q = c->q_dim, KV = c->kv_dim, H = c->hidden, V = c->vocab, S = c->seq;
    if (n_rows < 1 || n_rows > S || n_logit_rows < 0 || n_logit_rows > n_rows) return -1;
    for (int t = 0; t < n_rows; ++t) if (input[t] >= (uint32_t)V) return -2;
    int T = n_rows;
    float *x = (float *)malloc(sizeof(float) * (size_t)T * D);
    float *xn = (float *)malloc(sizeof(float) * (size_t)T * D);
    float *q = (float *)malloc(sizeof(float) * (size_t)T * Q);
    float *k = (float *)malloc(sizeof(float) * (size_t)T * KV);
    float *v = (float *)malloc(sizeof(float) * (size_t)T * KV);
    float *att = (float *)malloc(sizeof(float) * (size_t)T * Q);
    float *o = (float *)malloc(sizeof(float) * (size_t)T * D);
    float *h1 = (float *)malloc(sizeof(float) * (size_t)T * H);
    float *h3 = (float *)malloc(sizeof(float) * (size_t)T * H);
    orc_embedding(m->embed, D, input, T, x);
    for (int l = 0; l < c->nlayers; ++l) {
        const orc_layer *w = &m->layers[l];
        #pragma omp parallel for schedule(static)
        for (int t = 0; t < T; ++t) orc_rmsnorm(x + (size_t)t * D, w->gamma1, xn + (size_t)t * D, D);
        orc_gemm_in_major(xn, T, D, w->wq, Q, q);
        orc_gemm_in_major(xn, T, D, w->wk, KV, k);
        orc_gemm_in_major(xn, T, D, w->wv, KV, v);
        #pragma omp parallel for schedule(static)
        for (int t = 0; t < T; ++t) {
            rope_rows(m, q + (size_t)t * Q, c->heads, t);
            rope_rows(m, k + (size_t)t * KV, c->kv_heads, t);
            float *kd = m->kc[l] + (size_t)t * KV, *vd = m->vc[l] + (size_t)t * KV;
            for (int d = 0; d < KV; ++d) {
                kd[d] = m->kv_round_bf16 ? bf16_round(k[(size_t)t * KV + d]) : k[(size_t)t * KV + d];
                vd[d] = m->kv_round_bf16 ? bf16_round(v[(size_t)t * KV + d]) : v[(size_t)t * KV + d];
            }
        }
        if (k_cf && v_cf) {
            float *kd = k_cf + (size_t)l * KV * S, *vd = v_cf + (size_t)l * KV * S;
            memset(kd, 0, sizeof(float) * (size_t)KV * S);
            memset(vd, 0, sizeof(float) * (size_t)KV * S);
            for (int t = 0; t < T; ++t)
                for (int d = 0; d < KV; ++d) {
                    kd[(size_t)d * S + t] = m->kc[l][(size_t)t * KV + d];
                    vd[(size_t)d * S + t] = m->vc[l][(size_t)t * KV + d];
                }
        }
        #pragma omp parallel
        {
            float *scores = (float *)malloc(sizeof(float) * S);
            #pragma omp for schedule(dynamic, 4)
            for (int t = 0; t < T; ++t)
                orc_attend_row(c, q + (size_t)t * Q, m->kc[l], m->vc[l], t + 1, att + (size_t)t * Q, scores);
            free(scores);
        }
        orc_gemm_in_major(att, T, Q, w->wo, D, o);
        #pragma omp parallel for schedule(static)
        for (int t = 0; t < T; ++t) {
            float *xr = x + (size_t)t * D;
            const float *orow = o + (size_t)t * D;
            for (int d = 0; d < D; ++d) xr[d] = xr[d] + m->alpha * orow[d];      /* x2 */
            orc_rmsnorm(xr, w->gamma2, xn + (size_t)t * D, D);
        }
        orc_gemm_in_major(xn, T, D, w->w1, H, h1);
        orc_gemm_in_major(xn, T, D, w->w3, H, h3);
        #pragma omp parallel for schedule(static)
        for (size_t i = 0; i < (size_t)T * H; ++i) h1[i] = gate_act(c->ffn_activation, h1[i], h3[i]);
        orc_gemm_out_major(h1, T, H, w->w2, D, o);
        #pragma omp parallel for schedule(static)
        for (size_t i = 0; i < (size_t)T * D; ++i) x[i] = x[i] + m->alpha * o[i];
    }
    if (n_logit_rows > 0 && logits_out) {
        int r0 = T - n_logit_rows;
        for (int t = r0; t < T; ++t) orc_rmsnorm(x + (size_t)t * D, m->gamma_final, xn + (size_t)t * D, D);
        orc_gemm_out_major(xn + (size_t)r0 * D, n_logit_rows, D, m->embed, V, logits_out);
        if (softcap > 0.0f)
            for (size_t i = 0; i < (size_t)n_logit_rows * V; ++i) logits_out[i] = softcap_f(logits_out[i], softcap);
        memcpy(m->xf_last, xn + (size_t)(T - 1) * D, sizeof(float) * D);
    }
    m->len = T;
    free(x); free(xn); free(q); free(k); free(v); free(att); free(o); free(h1); free(h3);
    return 0;
}

/* One cached step through the layers (lib.rs:513-634, the arithmetic of encode_layer):
 * writes K/V at slot = len, attends over len+1 rows, len += 1.  x_io: in = residual stream
 * input (embedding row), out = last layer's output. */
static int cached_layers(orc_model *m, float *x) {
    const orc_config *c = &m->cfg;
    int D = c->dim, Q = c->q_dim, KV = c->kv_dim, H = c->hidden;
    if (m->len >= c->seq) return -3;                           /* lib.rs:242-245 */
    int slot = m->len, attn_len = m->len + 1;
    float *xn = (float *)malloc(sizeof(float) * D);
    float *q = (float *)malloc(sizeof(float) * Q);
    float *k = (float *)malloc(sizeof(float) * KV);
    float *v = (float *)malloc(sizeof(float) * KV);
    float *att = (float *)malloc(sizeof(float) * Q);
    float *o = (float *)malloc(sizeof(float) * D);
    float *h1 = (float *)malloc(sizeof(float) * H);
    float *h3 = (float *)malloc(sizeof(float) * H);
    float *scores = (float *)malloc(sizeof(float) * c->seq);
    for (int l = 0; l < c->nlayers; ++l) {
        const orc_layer *w = &m->layers[l];
        orc_rmsnorm(x, w->gamma1, xn, D);
        orc_gemm_in_major(xn, 1, D, w->wq, Q, q);
        orc_gemm_in_major(xn, 1, D, w->wk, KV, k);
        orc_gemm_in_major(xn, 1, D, w->wv, KV, v);
        rope_rows(m, q, c->heads, slot);
        rope_rows(m, k, c->kv_heads, slot);
        for (int d = 0; d < KV; ++d) {
            m->kc[l][(size_t)slot * KV + d] = m->kv_round_bf16 ? bf16_round(k[d]) : k[d];
            m->vc[l][(size_t)slot * KV + d] = m->kv_round_bf16 ? bf16_round(v[d]) : v[d];
        }
        orc_attend_row(c, q, m->kc[l], m->vc[l], attn_len, att, scores);
        orc_gemm_in_major(att, 1, Q, w->wo, D, o);
        for (int d = 0; d < D; ++d) x[d] = x[d] + m->alpha * o[d];
        orc_rmsnorm(x, w->gamma2, xn, D);
        orc_gemm_in_major(xn, 1, D, w->w1, H, h1);
        orc_gemm_in_major(xn, 1, D, w->w3, H, h3);
        for (int i = 0; i < H; ++i) h1[i] = gate_act(c->ffn_activation, h1[i], h3[i]);
        orc_gemm_out_major(h1, 1, H, w->w2, D, o);
        for (int d = 0; d < D; ++d) x[d] = x[d] + m->alpha * o[d];
    }
    m->len += 1;
    free(xn); free(q); free(k); free(v); free(att); free(o); free(h1); free(h3); free(scores);
    return 0;
}

/* lib.rs:271-304 decode_token_from_id: layers only, returns the un-normed residual stream */
int orc_decode_token_from_id(orc_model *m, uint32_t token, float *x_out) {
    if (token >= (uint32_t)m->cfg.vocab) return -2;
    memcpy(x_out, m->embed + (size_t)token * m->cfg.dim, sizeof(float) * m->cfg.dim);
    return cached_layers(m, x_out);
}

/* lib.rs:239-269 decode_token: same, from a caller-supplied input vector */
int orc_decode_token(orc_model *m, const float *x_in, float *x_out) {
    memcpy(x_out, x_in, sizeof(float) * m->cfg.dim);
    return cached_layers(m, x_out);
}

/* decode.rs:91-127 decode_next_logits: layers, final RMSNorm, tied LM head, softcap.
 * With softcap = 0 these are the raw logits every GPU head kernel of lib.rs:1515-1723 reduces. */
int orc_decode_logits_from_id(orc_model *m, uint32_t token, float softcap, float *logits) {
    int D = m->cfg.dim, V = m->cfg.vocab;
    float *x = (float *)malloc(sizeof(float) * D);
    int rc = orc_decode_token_from_id(m, token, x);
    if (rc == 0) {
        orc_rmsnorm(x, m->gamma_final, m->xf_last, D);
        orc_gemm_out_major(m->xf_last, 1, D, m->embed, V, logits);
        if (softcap > 0.0f) for (int i = 0; i < V; ++i) logits[i] = softcap_f(logits[i], softcap);
    }
    free(x);
    return rc;
}

/* ------------------------------------------------------------------ heads */

/* lib.rs:1515-1565 + 1725-1760: max value, ties -> lower index */
uint32_t orc_argmax_lower(const float *logits, int n) {
    float best = -INFINITY; uint32_t bi = 0xffffffffu;
    for (int i = 0; i < n; ++i)
        if (logits[i] > best || (logits[i] == best && (uint32_t)i < bi)) { best = logits[i]; bi = (uint32_t)i; }
    return bi;
}

/* f32::total_cmp as a signed-integer key (inference.rs:778-783 uses Iterator::max_by(total_cmp),
 * which returns the LAST maximal element) */
static int32_t total_key(float f) {
    int32_t b; memcpy(&b, &f, 4);
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

uint32_t orc_argmax_last(const float *logits, int n) {
    if (n <= 0) return 0;
    int bi = 0; int32_t best = total_key(logits[0]);
    for (int i = 1; i < n; ++i) { int32_t kx = total_key(logits[i]); if (kx >= best) { best = kx; bi = i; } }
    return (uint32_t)bi;
}

/* lib.rs:1567-1635: per block of 256 rows, top_k rounds of (max value, lower index) selection;
 * exhausted blocks pad with (-inf, 0xffffffff).  Raw logits (no softcap, no temperature). */
void orc_block_topk(const float *logits, int V, int top_k, float *out_vals, uint32_t *out_idxs) {
    int B = (V + ORC_BLOCK - 1) / ORC_BLOCK;
    for (int b = 0; b < B; ++b) {
        float cand[ORC_BLOCK]; uint32_t cidx[ORC_BLOCK];
        for (int t = 0; t < ORC_BLOCK; ++t) {
            int row = b * ORC_BLOCK + t;
            if (row < V) { cand[t] = logits[row]; cidx[t] = (uint32_t)row; }
            else { cand[t] = -INFINITY; cidx[t] = 0xffffffffu; }
        }
        for (int r = 0; r < top_k; ++r) {
            float bv = cand[0]; uint32_t bi = cidx[0];
            for (int t = 1; t < ORC_BLOCK; ++t)
                if (cand[t] > bv || (cand[t] == bv && cidx[t] < bi)) { bv = cand[t]; bi = cidx[t]; }
            out_vals[b * top_k + r] = bv;
            out_idxs[b * top_k + r] = bi;
            for (int t = 0; t < ORC_BLOCK; ++t)
                if (cidx[t] == bi) { cand[t] = -INFINITY; cidx[t] = 0xffffffffu; }
        }
    }
}

/* decode.rs:218-253 merge_topk_candidates */
int orc_merge_topk(const float *vals, const uint32_t *idxs, int count, int top_k,
                   float *out_vals, uint32_t *out_idxs) {
    for (int i = 0; i < top_k; ++i) { out_vals[i] = -INFINITY; out_idxs[i] = 0xffffffffu; }
    for (int c = 0; c < count; ++c) {
        float val = vals[c]; uint32_t idx = idxs[c];
        if (idx == 0xffffffffu || !isfinite(val)) continue;
        int at = -1;
        for (int s = 0; s < top_k; ++s)
            if (val > out_vals[s] || (val == out_vals[s] && idx < out_idxs[s])) { at = s; break; }
        if (at >= 0) {
            for (int i = top_k - 1; i > at; --i) { out_vals[i] = out_vals[i - 1]; out_idxs[i] = out_idxs[i - 1]; }
            out_vals[at] = val; out_idxs[at] = idx;
        }
    }
    for (int i = 0; i < top_k; ++i) if (out_idxs[i] == 0xffffffffu) return i;
    return top_k;
}

/* decode.rs:133-165: block top-k, merge, softcap on the survivors */
int orc_topk_candidates(const float *raw_logits, int V, int top_k, float softcap,
                        uint32_t *out_idxs, float *out_vals) {
    if (top_k > ORC_MAX_TOPK) top_k = ORC_MAX_TOPK;
    if (top_k > V) top_k = V;
    int B = (V + ORC_BLOCK - 1) / ORC_BLOCK;
    float *bv = (float *)malloc(sizeof(float) * B * top_k);
    uint32_t *bi = (uint32_t *)malloc(sizeof(uint32_t) * B * top_k);
    orc_block_topk(raw_logits, V, top_k, bv, bi);
    int n = orc_merge_topk(bv, bi, B * top_k, top_k, out_vals, out_idxs);
    if (softcap > 0.0f) for (int i = 0; i < n; ++i) out_vals[i] = softcap * tanhf(out_vals[i] / softcap);
    free(bv); free(bi);
    return n;
}

/* lib.rs:1637-1700: z = softcap(logit) * inv_T; per block max and sum exp(z - max) */
void orc_block_stats(const float *raw_logits, int V, float inv_temperature, float softcap,
                     float *maxes, float *sums) {
    int B = (V + ORC_BLOCK - 1) / ORC_BLOCK;
    for (int b = 0; b < B; ++b) {
        int r0 = b * ORC_BLOCK, r1 = r0 + ORC_BLOCK < V ? r0 + ORC_BLOCK : V;
        float mx = -INFINITY;
        for (int r = r0; r < r1; ++r) { float z = softcap_f(raw_logits[r], softcap) * inv_temperature; if (z > mx) mx = z; }
        float s = 0.0f;
        for (int r = r0; r < r1; ++r) s += expf(softcap_f(raw_logits[r], softcap) * inv_temperature - mx);
        maxes[b] = mx; sums[b] = s;
    }
}

/* lib.rs:1702-1723 + 489-511: softcapped (not temperature-scaled) logits of one block */
int orc_materialize_block(const float *raw_logits, int V, int block_idx, float softcap, float *out) {
    int r0 = block_idx * ORC_BLOCK;
    int valid = V - r0; if (valid > ORC_BLOCK) valid = ORC_BLOCK; if (valid < 0) valid = 0;
    for (int i = 0; i < valid; ++i) out[i] = softcap_f(raw_logits[r0 + i], softcap);
    return valid;
}

/* ------------------------------------------------------------------ RNG and samplers */

/* inference.rs:759-764 */
uint64_t orc_next_u64(uint64_t *state) {
    *state = *state * 6364136223846793005ull + 1442695040888963407ull;
    return *state;
}
/* inference.rs:766-768 */
float orc_next_f32(uint64_t *state) {
    return (float)(orc_next_u64(state) >> 40) / (float)(1ull << 24);
}

/* inference.rs:893-917 */
size_t orc_sample_softmax_index(const float *logits, int n, float temperature, uint64_t *rng) {
    float mx = -INFINITY;
    for (int i = 0; i < n; ++i) mx = fmaxf(mx, logits[i]);
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) sum += expf((logits[i] - mx) / temperature);
    if (!isfinite(sum) || sum <= 0.0f) return orc_argmax_last(logits, n);
    float draw = orc_next_f32(rng) * sum;
    for (int i = 0; i < n; ++i) {
        draw -= expf((logits[i] - mx) / temperature);
        if (draw <= 0.0f) return (size_t)i;
    }
    return n > 0 ? (size_t)(n - 1) : 0;
}

typedef struct { int32_t key; int idx; } orc_kv;
static int cmp_desc(const void *a, const void *b) {
    const orc_kv *x = (const orc_kv *)a, *y = (const orc_kv *)b;
    if (x->key != y->key) return x->key < y->key ? 1 : -1;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);   /* unstable in the reference; index asc here */
}

/* inference.rs:770-821 */
uint32_t orc_sample_next(const float *logits, int n, float temperature, int top_k, uint64_t *rng) {
    if (temperature <= 0.0f || top_k == 1) return orc_argmax_last(logits, n);
    if (top_k == 0 || top_k >= n) return (uint32_t)orc_sample_softmax_index(logits, n, temperature, rng);
    orc_kv *ix = (orc_kv *)malloc(sizeof(orc_kv) * n);
    for (int i = 0; i < n; ++i) { ix[i].key = total_key(logits[i]); ix[i].idx = i; }
    qsort(ix, n, sizeof(orc_kv), cmp_desc);
    int kk = top_k < n ? top_k : n;
    float mx = -INFINITY;
    for (int i = 0; i < kk; ++i) mx = fmaxf(mx, logits[ix[i].idx]);
    float sum = 0.0f;
    for (int i = 0; i < kk; ++i) sum += expf((logits[ix[i].idx] - mx) / temperature);
    uint32_t res;
    if (!isfinite(sum) || sum <= 0.0f) { res = (uint32_t)ix[0].idx; free(ix); return res; }
    float draw = orc_next_f32(rng) * sum;
    for (int i = 0; i < kk; ++i) {
        draw -= expf((logits[ix[i].idx] - mx) / temperature);
        if (draw <= 0.0f) { res = (uint32_t)ix[i].idx; free(ix); return res; }
    }
    res = (uint32_t)ix[kk - 1].idx; free(ix); return res;
}

/* inference.rs:823-849 */
uint32_t orc_sample_topk_candidates(const uint32_t *idxs, const float *logits, int n,
                                    float temperature, uint64_t *rng) {
    if (n <= 0) return 0;
    if (temperature <= 0.0f || n == 1) return idxs[0];
    float mx = -INFINITY;
    for (int i = 0; i < n; ++i) mx = fmaxf(mx, logits[i]);
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) sum += expf((logits[i] - mx) / temperature);
    if (!isfinite(sum) || sum <= 0.0f) return idxs[0];
    float draw = orc_next_f32(rng) * sum;
    for (int i = 0; i < n; ++i) {
        draw -= expf((logits[i] - mx) / temperature);
        if (draw <= 0.0f) return idxs[i];
    }
    return idxs[n - 1];
}

/* inference.rs:851-891 */
size_t orc_sample_block_from_stats(const float *maxes, const float *sums, int B, uint64_t *rng) {
    if (B <= 0) return 0;
    float g = -INFINITY;
    for (int b = 0; b < B; ++b) if (isfinite(maxes[b])) g = fmaxf(g, maxes[b]);
    if (!isfinite(g)) return 0;
    float total = 0.0f;
    for (int b = 0; b < B; ++b) {
        float w = (isfinite(maxes[b]) && isfinite(sums[b]) && sums[b] > 0.0f) ? expf(maxes[b] - g) * sums[b] : 0.0f;
        total += w;
    }
    if (!isfinite(total) || total <= 0.0f) return 0;
    float draw = orc_next_f32(rng) * total;
    for (int b = 0; b < B; ++b) {
        float w = (isfinite(maxes[b]) && isfinite(sums[b]) && sums[b] > 0.0f) ? expf(maxes[b] - g) * sums[b] : 0.0f;
        draw -= w;
        if (draw <= 0.0f) return (size_t)b;
    }
    return (size_t)(B - 1);
}

/* inference.rs:919-921 */
uint32_t orc_sample_block_logits(uint32_t base, const float *logits, int n, float temperature, uint64_t *rng) {
    return base + (uint32_t)orc_sample_softmax_index(logits, n, temperature, rng);
}

/* ------------------------------------------------------------------ token loops */

/* inference.rs:751-757 */
int orc_fill_input_window(const uint32_t *generated, int n, int seq, uint32_t *input) {
    memset(input, 0, sizeof(uint32_t) * seq);
    int start = n > seq ? n - seq : 0;
    int cnt = n - start;
    memcpy(input, generated + start, sizeof(uint32_t) * cnt);
    return cnt;
}

/* inference.rs:687-734 run_naive_sample (the reference's CPU-side loop; each step re-runs the
 * window forward).  generated: in = prompt (n_prompt ids), capacity n_prompt + steps.
 * prompt_logits are the logits of the prompt's last position. */
int orc_run_naive_sample(orc_model *m, uint32_t *generated, int n_prompt, const float *prompt_logits,
                         float softcap, int steps, float temperature, int top_k, uint64_t seed,
                         uint32_t *sampled) {
    int V = m->cfg.vocab, S = m->cfg.seq;
    uint64_t rng = seed;
    int n = n_prompt;
    if (steps <= 0) return 0;
    uint32_t next = orc_sample_next(prompt_logits, V, temperature, top_k, &rng);
    generated[n++] = next; sampled[0] = next;
    uint32_t *input = (uint32_t *)malloc(sizeof(uint32_t) * S);
    float *logits = (float *)malloc(sizeof(float) * V);
    for (int i = 1; i < steps; ++i) {
        int ctx = orc_fill_input_window(generated, n, S, input);
        int rc = orc_forward_window(m, input, ctx, softcap, 1, logits, NULL, NULL);
        if (rc) { free(input); free(logits); return rc; }
        next = orc_sample_next(logits, V, temperature, top_k, &rng);
        generated[n++] = next; sampled[i] = next;
    }
    free(input); free(logits);
    return 0;
}

/* inference.rs:542-648 run_cached_sample, with the KV cache already holding the prompt
 * (len = live prompt length): suffix tokens through the token loop, first sample from the
 * prompt logits on the host, then the branch chosen once from (temperature, top_k). */
int orc_run_cached_sample(orc_model *m, uint32_t *generated, int n_prompt, const float *prompt_logits,
                          const uint32_t *suffix, int n_suffix, float softcap, int steps,
                          float temperature, int top_k, uint64_t seed, uint32_t *sampled) {
    int V = m->cfg.vocab;
    uint64_t rng = seed;
    int n = n_prompt, rc = 0;
    float *logits = (float *)malloc(sizeof(float) * V);
    for (int i = 0; i < n_suffix && !rc; ++i) rc = orc_decode_logits_from_id(m, suffix[i], softcap, logits);
    if (rc || steps <= 0) { free(logits); return rc; }
    uint32_t cur = orc_sample_next(prompt_logits, V, temperature, top_k, &rng);
    generated[n++] = cur; sampled[0] = cur;
    int B = (V + ORC_BLOCK - 1) / ORC_BLOCK;
    float *maxes = (float *)malloc(sizeof(float) * B), *sums = (float *)malloc(sizeof(float) * B);
    float blk[ORC_BLOCK], cv[ORC_MAX_TOPK]; uint32_t ci[ORC_MAX_TOPK];
    for (int i = 1; i < steps && !rc; ++i) {
        uint32_t next;
        if (temperature <= 0.0f || top_k == 1) {                        /* inference.rs:576-585 */
            rc = orc_decode_logits_from_id(m, cur, 0.0f, logits);
            next = orc_argmax_lower(logits, V);
        } else if (top_k > 0 && top_k <= ORC_MAX_TOPK) {                /* :586-599 */
            rc = orc_decode_logits_from_id(m, cur, 0.0f, logits);
            int nc = orc_topk_candidates(logits, V, top_k, softcap, ci, cv);
            next = orc_sample_topk_candidates(ci, cv, nc, temperature, &rng);
        } else if (top_k == 0) {                                        /* :600-625 */
            rc = orc_decode_logits_from_id(m, cur, 0.0f, logits);
            float inv_t = 1.0f / fmaxf(temperature, 1.17549435e-38f);   /* decode.rs:174 */
            orc_block_stats(logits, V, inv_t, softcap, maxes, sums);
            size_t b = orc_sample_block_from_stats(maxes, sums, B, &rng);
            int valid = orc_materialize_block(logits, V, (int)b, softcap, blk);
            next = orc_sample_block_logits((uint32_t)(b * ORC_BLOCK), blk, valid, temperature, &rng);
        } else {                                                        /* :626-638 */
            rc = orc_decode_logits_from_id(m, cur, softcap, logits);
            next = orc_sample_next(logits, V, temperature, top_k, &rng);
        }
        generated[n++] = next; sampled[i] = next; cur = next;
    }
    free(logits); free(maxes); free(sums);
    return rc;
}

/* ------------------------------------------------------------------ weight-format restatements
 * The 8-bit and 4-bit weight streams are this build's own formats (the reference is fp32 only);
 * the oracle restates them so that the device's stored weights can be checked bit for bit and
 * so that quantised configs are compared against the DEQUANTISED weights.                    */

/* OCP FP8 E4M3 (e4m3fn: bias 7, max 448, no inf, S.1111.111 = NaN), round to nearest even,
 * saturating.  Returns the byte. */
uint8_t orc_f32_to_e4m3(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    float a = fabsf(f);
    if (a != a) return sign | 0x7f;
    if (a >= 464.0f) return sign | 0x7e;                 /* >= halfway past 448 saturates to 448 */
    if (a < 0.0009765625f) return sign;                  /* < 2^-10 (half of min subnormal 2^-9) -> 0 */
    int e; float mant = frexpf(a, &e);                   /* a = mant * 2^e, mant in [0.5,1) */
    int exp = e - 1;                                     /* a = (2*mant) * 2^exp */
    if (exp < -6) {                                      /* subnormal: units of 2^-9 */
        float q = a * 512.0f;
        float r = nearbyintf(q);                         /* RNE in default rounding mode */
        int qi = (int)r;
        if (qi >= 8) return sign | 0x08;                 /* rounds up to min normal */
        return sign | (uint8_t)qi;
    }
    float frac = (2.0f * mant - 1.0f) * 8.0f;            /* [0,8) */
    float r = nearbyintf(frac);
    int mi = (int)r;
    if (mi == 8) { mi = 0; exp += 1; }
    if (exp > 8 || (exp == 8 && mi > 6)) return sign | 0x7e;
    return sign | (uint8_t)(((exp + 7) << 3) | mi);
}

float orc_e4m3_to_f32(uint8_t b) {
    int s = b >> 7, e = (b >> 3) & 0xf, m = b & 7;
    float v;
    if (e == 0xf && m == 7) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return s ? -v : v;
}

/* Per-output-channel FP8: W is out-major [O][K] fp32; scale[o] = amax_o / 448 (fp32; 1.0 when
 * the row is all zero); q = e4m3(w / scale); dequant = q * scale. */
void orc_quant_fp8_rows(const float *W, int O, int K, uint8_t *q, float *scale, float *dequant) {
    #pragma omp parallel for schedule(static)
    for (int o = 0; o < O; ++o) {
        const float *w = W + (size_t)o * K;
        float amax = 0.0f;
        for (int k = 0; k < K; ++k) amax = fmaxf(amax, fabsf(w[k]));
        float s = amax > 0.0f ? amax / 448.0f : 1.0f;
        if (scale) scale[o] = s;
        for (int k = 0; k < K; ++k) {
            uint8_t b = orc_f32_to_e4m3(w[k] / s);
            if (q) q[(size_t)o * K + k] = b;
            if (dequant) dequant[(size_t)o * K + k] = orc_e4m3_to_f32(b) * s;
        }
    }
}

/* 4-bit symmetric, groups of 128 along K: scale = bf16(amax_g / 7) (1.0 when the group is all
 * zero); q = clamp(rne(w / scale), -8, 7); dequant = q * scale.  q is returned as int8. */
void orc_quant_int4_g128(const float *W, int O, int K, int8_t *q, float *scale, float *dequant) {
    int G = (K + 127) / 128;
    #pragma omp parallel for schedule(static)
    for (int o = 0; o < O; ++o)
        for (int g = 0; g < G; ++g) {
            int k0 = g * 128, k1 = k0 + 128 < K ? k0 + 128 : K;
            const float *w = W + (size_t)o * K;
            float amax = 0.0f;
            for (int k = k0; k < k1; ++k) amax = fmaxf(amax, fabsf(w[k]));
            float s = amax > 0.0f ? bf16_round(amax / 7.0f) : 1.0f;
            if (scale) scale[(size_t)o * G + g] = s;
            for (int k = k0; k < k1; ++k) {
                float r = nearbyintf(w[k] / s);
                if (r > 7.0f) r = 7.0f;
                if (r < -8.0f) r = -8.0f;
                if (q) q[(size_t)o * K + k] = (int8_t)r;
                if (dequant) dequant[(size_t)o * K + k] = r * s;
            }
        }
}

/* transpose helper: in-major [K][O] -> out-major [O][K] */
void orc_transpose(const float *in, int rows, int cols, float *out) {
    #pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c) out[(size_t)c * rows + r] = in[(size_t)r * cols + c];
}
