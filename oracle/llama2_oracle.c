/*
 * TEST INFRASTRUCTURE - NOT PRODUCT CODE.
 *
 * CPU restatement of the reference's llama2-style fp32 forward pass, used only
 * as (a) the parity checker for the HIP decode engine and (b) the timed CPU
 * baseline.  Nothing in the shipped library links or calls this file.
 *
 * Each routine follows the arithmetic order of the reference routine it cites
 * (all paths relative to the reference tree, directory
 * CudaExtension.llm32.llama2/Files/):
 *
 *   orc_rmsnorm          llama2_cpu.cpp:189-202   (rmsnorm)
 *   orc_softmax          llama2_cpu.cpp:204-222   (softmax)
 *   orc_matvec           llama2_cpu.cpp:224-236   (matmul, omp over rows)
 *   orc_rope_pairs       llama2_cpu.cpp:238-262   (rope, adjacent-pair form)
 *   orc_freq_tables      llama2_cpu.cpp:388-414   (precompute_freqs_cis)
 *   orc_llama_forward    llama2_cpu.cpp:264-386   (TransformerCpu::forward)
 *   orc_argmax           llama2_sampler.cpp:25-36 (sample_argmax, first max wins)
 *   weight blob order    llama2_cpu.cpp:74-106    (memory_map_weights)
 *
 * fp32 everywhere, sums run left to right exactly as the reference's loops do,
 * so single-thread results are reproducible bit for bit; the OpenMP pragmas sit
 * on the same two loops as in the reference (matvec rows, attention heads) and
 * do not change any summation order.
 *
 * Parity pins (see tests/test_oracle_*.py): softmax vs scipy.special.softmax,
 * rmsnorm vs torch.nn.functional.rms_norm, matvec vs numpy, RoPE vs complex
 * multiplication by exp(i*pos*theta^(-2j/hs)), the whole forward vs
 * transformers.LlamaForCausalLM (independent library implementation, full
 * sequence, fp64) and argmax vs the first-max rule.  The reference's own C++
 * for this path includes <io.h> and the CUDA headers (llama2_cpu.h:6,22 via
 * primitives.h:20-27) and so cannot be compiled in this image without
 * stand-ins; no oracle/_ref build exists for it.
 *
 * One checker-only option has no counterpart in the reference: orc_set_kv_bf16(1)
 * makes the forward round the rotated key and the value of the current position
 * to bfloat16 (round to nearest even) before they enter the cache and the
 * attention, which is what the HIP engine's 16-bit cache mode does.  The
 * rounding (orc_round_bf16) is pinned against torch's float32 -> bfloat16
 * conversion, ties, denormals and infinities included.
 */
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    int dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
} OrcConfig;

typedef struct {
    OrcConfig cfg;
    /* weights: pointers into one caller-owned fp32 blob */
    const float *rms_att, *rms_ffn, *rms_final, *tok_emb;
    const float *wq, *wk, *wv, *wo, *w1, *w2, *w3, *wcls;
    /* run state */
    float *x, *xb, *xb2, *hb, *hb2, *q, *k, *v, *att, *logits;
    float *kcache, *vcache, *fcos, *fsin;
} OrcLlama;

/* checker-only: cache entries rounded to bfloat16 (see the header) */
static int g_kv_bf16 = 0;
void orc_set_kv_bf16(int on) { g_kv_bf16 = on; }

/* fp32 -> nearest bfloat16 (ties to even), returned as fp32; NaN stays NaN */
void orc_round_bf16(float *x, int n)
{
    for (int i = 0; i < n; i++) {
        uint32_t u;
        memcpy(&u, &x[i], 4);
        if ((u & 0x7fffffffu) > 0x7f800000u)
            u |= 0x00400000u;
        else
            u += 0x7fffu + ((u >> 16) & 1u);
        u &= 0xffff0000u;
        memcpy(&x[i], &u, 4);
    }
}

/* worker threads of the parallel loops below (the reference takes OpenMP's default); returns the previous limit */
int orc_set_threads(int n)
{
#ifdef _OPENMP
    int prev = omp_get_max_threads();
    if (n > 0) omp_set_num_threads(n);
    return prev;
#else
    (void)n;
    return 1;
#endif
}

void orc_rmsnorm(float *o, const float *x, const float *w, int n)
{
    float ss = 0.0f;
    for (int j = 0; j < n; j++)
        ss += x[j] * x[j];
    ss /= n;
    ss += 1e-5f;
    ss = 1.0f / sqrtf(ss);
    for (int j = 0; j < n; j++)
        o[j] = w[j] * (ss * x[j]);
}

void orc_softmax(float *x, int n)
{
    float mx = x[0];
    for (int i = 1; i < n; i++)
        if (x[i] > mx)
            mx = x[i];
    float sum = 0.0f;
    for (int i = 0; i < n; i++) {
        x[i] = expf(x[i] - mx);
        sum += x[i];
    }
    for (int i = 0; i < n; i++)
        x[i] /= sum;
}

/* out[d] = W[d,n] . x[n], W row-major */
void orc_matvec(float *out, const float *x, const float *w, int n, int d)
{
    int i;
#pragma omp parallel for private(i)
    for (i = 0; i < d; i++) {
        float acc = 0.0f;
        const float *row = w + (size_t)i * n;
        for (int j = 0; j < n; j++)
            acc += row[j] * x[j];
        out[i] = acc;
    }
}

/* rotate adjacent (even, odd) pairs of every head of q and k by the table row
 * that starts at fcos/fsin + off */
void orc_rope_pairs(int n_heads, int hs, float *q, float *k, const float *fcos,
                    const float *fsin, int off)
{
    fcos += off;
    fsin += off;
    for (int h = 0; h < n_heads; h++) {
        float *qh = q + h * hs, *kh = k + h * hs;
        for (int i = 0; i < hs; i += 2) {
            float c = fcos[i / 2], s = fsin[i / 2];
            float q0 = qh[i], q1 = qh[i + 1], k0 = kh[i], k1 = kh[i + 1];
            qh[i] = q0 * c - q1 * s;
            qh[i + 1] = q0 * s + q1 * c;
            kh[i] = k0 * c - k1 * s;
            kh[i + 1] = k0 * s + k1 * c;
        }
    }
}

/* tables [pos][hs/2]: cos/sin(pos * theta^(-i/hs)), i even, theta = 10000 */
void orc_freq_tables(int hs, int seq_len, float *fcos, float *fsin)
{
    const float theta = 10000.0f;
    int half = hs / 2;
    float *fr = (float *)calloc(half, sizeof(float));
    for (int i = 0; i < hs; i += 2) {
        float e = i / (float)hs;
        float d = powf(theta, e);
        fr[i / 2] = (d == 0.0) ? 0 : 1.0f / d;
    }
    for (size_t p = 0; p < (size_t)seq_len; p++)
        for (int j = 0; j < half; j++) {
            fcos[p * hs / 2 + j] = cosf(p * fr[j]);
            fsin[p * hs / 2 + j] = sinf(p * fr[j]);
        }
    free(fr);
}

int orc_argmax(const float *p, int n)
{
    int best = 0;
    float bv = p[0];
    for (int i = 1; i < n; i++)
        if (p[i] > bv) {
            best = i;
            bv = p[i];
        }
    return best;
}

/* number of floats the weight blob must hold */
size_t orc_llama_weight_count(const OrcConfig *c, int shared_classifier)
{
    size_t L = c->n_layers, dim = c->dim, hid = c->hidden_dim;
    size_t hs = dim / c->n_heads, kvd = hs * c->n_kv_heads;
    size_t n = 2 * L * dim + dim + (size_t)c->vocab_size * dim;
    n += L * dim * dim + 2 * L * dim * kvd + L * dim * dim + 3 * L * dim * hid;
    if (!shared_classifier)
        n += (size_t)c->vocab_size * dim;
    return n;
}

OrcLlama *orc_llama_create(const OrcConfig *c, const float *blob, int shared_classifier)
{
    OrcLlama *m = (OrcLlama *)calloc(1, sizeof(OrcLlama));
    if (!m)
        return NULL;
    m->cfg = *c;
    size_t L = c->n_layers, dim = c->dim, hid = c->hidden_dim;
    size_t hs = dim / c->n_heads, kvd = hs * c->n_kv_heads;
    const float *p = blob;
    m->rms_att = p;   p += L * dim;
    m->rms_ffn = p;   p += L * dim;
    m->rms_final = p; p += dim;
    m->tok_emb = p;   p += (size_t)c->vocab_size * dim;
    m->wq = p;        p += L * dim * dim;
    m->wk = p;        p += L * dim * kvd;
    m->wv = p;        p += L * dim * kvd;
    m->wo = p;        p += L * dim * dim;
    m->w1 = p;        p += L * dim * hid;
    m->w2 = p;        p += L * hid * dim;
    m->w3 = p;        p += L * dim * hid;
    m->wcls = shared_classifier ? m->tok_emb : p;

    m->x = (float *)calloc(dim, 4);
    m->xb = (float *)calloc(dim, 4);
    m->xb2 = (float *)calloc(dim, 4);
    m->hb = (float *)calloc(hid, 4);
    m->hb2 = (float *)calloc(hid, 4);
    m->q = (float *)calloc(dim, 4);
    /* the reference sizes k and v as kv_dim floats but its rope loop walks all
     * n_heads heads of k (llama2_cpu.cpp:238-262), which overruns the buffer
     * when n_kv_heads < n_heads; dim floats keep that walk inside the buffer
     * (the extra heads are never read back) */
    m->k = (float *)calloc(dim, 4);
    m->v = (float *)calloc(dim, 4);
    m->att = (float *)calloc((size_t)c->n_heads * c->seq_len, 4);
    m->logits = (float *)calloc(c->vocab_size, 4);
    m->kcache = (float *)calloc(L * c->seq_len * kvd, 4);
    m->vcache = (float *)calloc(L * c->seq_len * kvd, 4);
    m->fcos = (float *)calloc((size_t)c->seq_len * (hs / 2), 4);
    m->fsin = (float *)calloc((size_t)c->seq_len * (hs / 2), 4);
    orc_freq_tables((int)hs, c->seq_len, m->fcos, m->fsin);
    return m;
}

void orc_llama_destroy(OrcLlama *m)
{
    if (!m)
        return;
    free(m->x); free(m->xb); free(m->xb2); free(m->hb); free(m->hb2);
    free(m->q); free(m->k); free(m->v); free(m->att); free(m->logits);
    free(m->kcache); free(m->vcache); free(m->fcos); free(m->fsin);
    free(m);
}

/* one decode step; returns a pointer to vocab_size logits owned by the model */
float *orc_llama_forward(OrcLlama *m, int token, int pos)
{
    const OrcConfig *c = &m->cfg;
    int dim = c->dim, hid = c->hidden_dim;
    int hs = dim / c->n_heads;
    int kvd = (dim * c->n_kv_heads) / c->n_heads;
    int kv_mul = c->n_heads / c->n_kv_heads;
    float *x = m->x;

    memcpy(x, m->tok_emb + (size_t)token * dim, dim * sizeof(float));
    int foff = pos * hs / 2;

    for (size_t l = 0; l < (size_t)c->n_layers; l++) {
        orc_rmsnorm(m->xb, x, m->rms_att + l * dim, dim);

        orc_matvec(m->q, m->xb, m->wq + l * dim * dim, dim, dim);
        orc_matvec(m->k, m->xb, m->wk + l * dim * kvd, dim, kvd);
        orc_matvec(m->v, m->xb, m->wv + l * dim * kvd, dim, kvd);

        orc_rope_pairs(c->n_heads, hs, m->q, m->k, m->fcos, m->fsin, foff);

        if (g_kv_bf16) {
            orc_round_bf16(m->k, kvd);
            orc_round_bf16(m->v, kvd);
        }
        size_t loff = l * c->seq_len * kvd;
        memcpy(m->kcache + loff + (size_t)pos * kvd, m->k, kvd * sizeof(float));
        memcpy(m->vcache + loff + (size_t)pos * kvd, m->v, kvd * sizeof(float));

        int h;
#pragma omp parallel for private(h)
        for (h = 0; h < c->n_heads; h++) {
            const float *qh = m->q + h * hs;
            float *att = m->att + (size_t)h * c->seq_len;
            for (int t = 0; t <= pos; t++) {
                const float *kt = m->kcache + loff + (size_t)t * kvd + (h / kv_mul) * hs;
                float s = 0.0f;
                for (int i = 0; i < hs; i++)
                    s += qh[i] * kt[i];
                s /= sqrtf((float)hs);
                att[t] = s;
            }
            orc_softmax(att, pos + 1);
            float *o = m->xb + h * hs;
            memset(o, 0, hs * sizeof(float));
            for (int t = 0; t <= pos; t++) {
                const float *vt = m->vcache + loff + (size_t)t * kvd + (h / kv_mul) * hs;
                float a = att[t];
                for (int i = 0; i < hs; i++)
                    o[i] += a * vt[i];
            }
        }

        orc_matvec(m->xb2, m->xb, m->wo + l * dim * dim, dim, dim);
        for (int i = 0; i < dim; i++)
            x[i] += m->xb2[i];

        orc_rmsnorm(m->xb, x, m->rms_ffn + l * dim, dim);
        orc_matvec(m->hb, m->xb, m->w1 + l * dim * hid, dim, hid);
        orc_matvec(m->hb2, m->xb, m->w3 + l * dim * hid, dim, hid);
        for (int i = 0; i < hid; i++) {
            float g = m->hb[i];
            g *= (1.0f / (1.0f + expf(-g)));
            g *= m->hb2[i];
            m->hb[i] = g;
        }
        orc_matvec(m->xb, m->hb, m->w2 + l * dim * hid, hid, dim);
        for (int i = 0; i < dim; i++)
            x[i] += m->xb[i];
    }

    orc_rmsnorm(x, x, m->rms_final, dim);
    orc_matvec(m->logits, x, m->wcls, dim, c->vocab_size);
    return m->logits;
}

/*
 * Greedy generation with the control flow of the reference's generate loop
 * (llm.cpp:184-265) for a prompt given as token ids: the prompt ids are forced
 * through positions 0..n_prompt-1, after which each step feeds back the argmax
 * of the previous step.  out_ids[pos] receives the token sampled AFTER position
 * pos (the prediction for pos+1); if all_logits is non-NULL it receives every
 * step's vocab_size logits.  No EOS stop: the caller asks for a fixed length.
 * Returns the number of steps run.
 */
int orc_llama_generate_greedy(OrcLlama *m, const int *prompt, int n_prompt, int n_steps,
                              int *out_ids, float *all_logits)
{
    int next = 0;
    for (int pos = 0; pos < n_steps; pos++) {
        int token = pos < n_prompt ? prompt[pos] : next;
        float *lg = orc_llama_forward(m, token, pos);
        next = orc_argmax(lg, m->cfg.vocab_size);
        out_ids[pos] = next;
        if (all_logits)
            memcpy(all_logits + (size_t)pos * m->cfg.vocab_size, lg,
                   m->cfg.vocab_size * sizeof(float));
    }
    return n_steps;
}

/* ---------------------------------------------------------------------------
 * Sampler (llama2_sampler.cpp): temperature, softmax, a 24-bit coin from xorshift64*, then either the inverse CDF over
 * all tokens or nucleus (top-p) sampling.  All accumulations are sequential fp32, as there.
 */
unsigned int orc_random_u32(unsigned long long *state)   /* llama2_sampler.cpp:115-121 */
{
    *state ^= *state >> 12;
    *state ^= *state << 25;
    *state ^= *state >> 27;
    return (unsigned int)((*state * 0x2545F4914F6CDD1Dull) >> 32);
}

float orc_random_f32(unsigned long long *state)          /* llama2_sampler.cpp:122-124: [0, 1) in steps of 2^-24 */
{
    return (orc_random_u32(state) >> 8) / 16777216.0f;
}

int orc_sample_mult(const float *p, int n, float coin)   /* llama2_sampler.cpp:38-49 */
{
    float cdf = 0.0f;
    for (int i = 0; i < n; i++) {
        cdf += p[i];
        if (coin < cdf) return i;
    }
    return n - 1;
}

typedef struct { float prob; int index; } OrcProbIndex;

/* descending by probability; equal probabilities keep the lower index first (the reference's qsort leaves their
 * order to the C library) */
static int orc_cmp_prob(const void *a, const void *b)
{
    const OrcProbIndex *x = (const OrcProbIndex *)a, *y = (const OrcProbIndex *)b;
    if (x->prob > y->prob) return -1;
    if (x->prob < y->prob) return 1;
    return (x->index > y->index) - (x->index < y->index);
}

int orc_sample_topp(const float *p, int n, float topp, float coin)   /* llama2_sampler.cpp:59-100 */
{
    OrcProbIndex *pi = (OrcProbIndex *)malloc((size_t)n * sizeof(OrcProbIndex));
    int n0 = 0;
    const float cutoff = (1.0f - topp) / (n - 1);
    for (int i = 0; i < n; i++)
        if (p[i] >= cutoff) { pi[n0].index = i; pi[n0].prob = p[i]; n0++; }
    qsort(pi, n0, sizeof(OrcProbIndex), orc_cmp_prob);
    float cum = 0.0f;
    int last = n0 - 1;
    for (int i = 0; i < n0; i++) {
        cum += pi[i].prob;
        if (cum > topp) { last = i; break; }
    }
    const float r = coin * cum;
    float cdf = 0.0f;
    int res = pi[last].index;
    for (int i = 0; i <= last; i++) {
        cdf += pi[i].prob;
        if (r < cdf) { res = pi[i].index; break; }
    }
    free(pi);
    return res;
}

/* sample (llama2_sampler.cpp:126-151); logits are overwritten with the probabilities when temperature != 0 */
int orc_sample(float *logits, int n, float temperature, float topp, unsigned long long *state)
{
    if (temperature == 0.0f) return orc_argmax(logits, n);
    for (int q = 0; q < n; q++) logits[q] /= temperature;
    orc_softmax(logits, n);
    const float coin = orc_random_f32(state);
    if (topp <= 0 || topp >= 1) return orc_sample_mult(logits, n, coin);
    return orc_sample_topp(logits, n, topp, coin);
}

/* generate loop of llm.cpp:208-245 with the sampler: sample() runs at every position, prompt positions included (its
 * result is discarded there but the random state advances). */
int orc_llama_generate_sampled(OrcLlama *m, const int *prompt, int n_prompt, int n_steps, float temperature, float topp,
                               unsigned long long *state, int *out_ids)
{
    int next = 0;
    for (int pos = 0; pos < n_steps; pos++) {
        int token = pos < n_prompt ? prompt[pos] : next;
        float *lg = orc_llama_forward(m, token, pos);
        next = orc_sample(lg, m->cfg.vocab_size, temperature, topp, state);
        out_ids[pos] = next;
    }
    return n_steps;
}
