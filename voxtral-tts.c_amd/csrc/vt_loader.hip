/*
 * vt_loader.hip - checkpoint file -> device (the on-disk format either side of the upload
 * entry points).  Reads a .safetensors file the way the reference does
 * (voxtral_tts_safetensors.c:204-405: 8-byte little-endian header length, a JSON object of
 * name -> {dtype, shape, data_offsets}, then the raw tensor bytes, mapped read-only) and
 * hands the tensors the reference looks up by name (voxtral_tts_llm.c:45-100,
 * voxtral_tts_acoustic.c:40-130, voxtral_tts_voice.c:251-290) to the upload entry points.
 * bf16 matrices are uploaded straight from the mapping; norm vectors, which checkpoints
 * hold as bf16, f16 or f32, are widened to f32 first like the reference's load_f32.
 *
 * Host code only; the JSON reader below understands exactly the flat header that the format
 * defines (string keys, objects with "dtype", "shape", "data_offsets"; "__metadata__" is
 * skipped).
 */
#include "vt_state.h"

#include <fcntl.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

struct st_tensor {
    char name[160];
    char dtype[8];
    int rank;
    long long shape[4];
    long long begin, end;         /* byte range inside the data section */
};

struct st_file {
    int fd;
    unsigned char *map;
    size_t size;
    size_t data0;                 /* offset of the data section */
    st_tensor *t;
    int n;
};

/* ---- header reader ------------------------------------------------------------------ */

struct st_cur { const char *p, *end; };

static void st_ws(st_cur *c) { while (c->p < c->end && (*c->p == ' ' || *c->p == '\n' || *c->p == '\t' || *c->p == '\r')) c->p++; }
static int st_eat(st_cur *c, char ch) { st_ws(c); if (c->p < c->end && *c->p == ch) { c->p++; return 1; } return 0; }

/* string without escape processing beyond \" and \\ (tensor names have none) */
static int st_string(st_cur *c, char *out, size_t cap) {
    st_ws(c);
    if (c->p >= c->end || *c->p != '"') return -1;
    c->p++;
    size_t n = 0;
    while (c->p < c->end && *c->p != '"') {
        char ch = *c->p++;
        if (ch == '\\' && c->p < c->end) ch = *c->p++;
        if (out && n + 1 < cap) out[n++] = ch;
    }
    if (c->p >= c->end) return -1;
    c->p++;
    if (out) out[n] = 0;
    return 0;
}

/* decimal integer; the header is not NUL-terminated, so every character is checked against its end */
static int st_int(st_cur *c, long long *v) {
    st_ws(c);
    int neg = 0;
    if (c->p < c->end && *c->p == '-') { neg = 1; c->p++; }
    if (c->p >= c->end || *c->p < '0' || *c->p > '9') return -1;
    long long x = 0;
    while (c->p < c->end && *c->p >= '0' && *c->p <= '9') {
        if (x > (0x7fffffffffffffffLL - 9) / 10) return -1;          /* would not fit */
        x = x * 10 + (*c->p++ - '0');
    }
    *v = neg ? -x : x;
    return 0;
}

/* skips any JSON value; nesting beyond ST_MAX_DEPTH is refused (the recursion is on the C stack) */
#define ST_MAX_DEPTH 32
static int st_skip_at(st_cur *c, int depth) {
    st_ws(c);
    if (c->p >= c->end || depth > ST_MAX_DEPTH) return -1;
    if (*c->p == '"') return st_string(c, NULL, 0);
    if (*c->p == '{' || *c->p == '[') {
        const char open = *c->p, close = open == '{' ? '}' : ']';
        c->p++;
        if (st_eat(c, close)) return 0;
        for (;;) {
            if (open == '{') { if (st_string(c, NULL, 0) || !st_eat(c, ':')) return -1; }
            if (st_skip_at(c, depth + 1)) return -1;
            if (st_eat(c, ',')) continue;
            return st_eat(c, close) ? 0 : -1;
        }
    }
    while (c->p < c->end && *c->p != ',' && *c->p != '}' && *c->p != ']') c->p++;
    return 0;
}
static int st_skip(st_cur *c) { return st_skip_at(c, 0); }

static int st_entry(st_cur *c, st_tensor *t) {
    if (!st_eat(c, '{')) return -1;
    t->rank = 0;
    t->dtype[0] = 0;
    t->begin = t->end = -1;
    if (st_eat(c, '}')) return -1;
    for (;;) {
        char key[32];
        if (st_string(c, key, sizeof key) || !st_eat(c, ':')) return -1;
        if (!strcmp(key, "dtype")) {
            if (st_string(c, t->dtype, sizeof t->dtype)) return -1;
        } else if (!strcmp(key, "shape")) {
            if (!st_eat(c, '[')) return -1;
            if (!st_eat(c, ']')) {
                for (;;) {
                    long long v;
                    if (st_int(c, &v)) return -1;
                    if (t->rank < 4) t->shape[t->rank] = v;
                    t->rank++;
                    if (st_eat(c, ',')) continue;
                    if (!st_eat(c, ']')) return -1;
                    break;
                }
            }
        } else if (!strcmp(key, "data_offsets")) {
            if (!st_eat(c, '[') || st_int(c, &t->begin) || !st_eat(c, ',') || st_int(c, &t->end) || !st_eat(c, ']'))
                return -1;
        } else if (st_skip(c)) {
            return -1;
        }
        if (st_eat(c, ',')) continue;
        return st_eat(c, '}') ? 0 : -1;
    }
}

static void st_close(st_file *f) {
    if (f->map && f->map != (unsigned char *)MAP_FAILED) munmap(f->map, f->size);
    if (f->fd >= 0) close(f->fd);
    free(f->t);
    memset(f, 0, sizeof *f);
    f->fd = -1;
}

static int st_open(st_file *f, const char *path) {
    memset(f, 0, sizeof *f);
    f->fd = open(path, O_RDONLY);
    if (f->fd < 0) { vt_set_error("safetensors: cannot open %s", path); return -1; }
    struct stat sb;
    if (fstat(f->fd, &sb) || sb.st_size < 8) { vt_set_error("safetensors: %s is too short", path); st_close(f); return -1; }
    f->size = (size_t)sb.st_size;
    f->map = (unsigned char *)mmap(NULL, f->size, PROT_READ, MAP_PRIVATE, f->fd, 0);
    if (f->map == (unsigned char *)MAP_FAILED) { vt_set_error("safetensors: mmap of %s failed", path); f->map = NULL; st_close(f); return -1; }
    unsigned long long hlen = 0;
    for (int i = 7; i >= 0; i--) hlen = (hlen << 8) | f->map[i];
    if (hlen < 2 || hlen > f->size - 8) { vt_set_error("safetensors: bad header length in %s", path); st_close(f); return -1; }
    f->data0 = 8 + (size_t)hlen;
    st_cur c = {(const char *)f->map + 8, (const char *)f->map + f->data0};
    int cap = 512;
    f->t = (st_tensor *)malloc(sizeof(st_tensor) * cap);
    if (!f->t || !st_eat(&c, '{')) { vt_set_error("safetensors: header of %s is not an object", path); st_close(f); return -1; }
    if (!st_eat(&c, '}')) {
        for (;;) {
            char name[160];
            if (st_string(&c, name, sizeof name) || !st_eat(&c, ':')) goto bad;
            if (!strcmp(name, "__metadata__")) {
                if (st_skip(&c)) goto bad;
            } else {
                if (f->n == cap) {
                    cap *= 2;
                    st_tensor *nt = (st_tensor *)realloc(f->t, sizeof(st_tensor) * cap);
                    if (!nt) goto bad;
                    f->t = nt;
                }
                st_tensor *t = &f->t[f->n];
                if (st_entry(&c, t)) goto bad;
                if (t->begin < 0 || t->end < t->begin || (size_t)t->end > f->size - f->data0) goto bad;
                strncpy(t->name, name, sizeof t->name - 1);
                t->name[sizeof t->name - 1] = 0;
                f->n++;
            }
            if (st_eat(&c, ',')) continue;
            if (!st_eat(&c, '}')) goto bad;
            break;
        }
    }
    return 0;
bad:
    vt_set_error("safetensors: malformed header in %s", path);
    st_close(f);
    return -1;
}

static const st_tensor *st_find(const st_file *f, const char *name) {
    for (int i = 0; i < f->n; i++)
        if (!strcmp(f->t[i].name, name)) return &f->t[i];
    return NULL;
}

/* number of elements, or -1 for shapes that no tensor of this model has (rank above 4, a
 * negative extent, a product beyond 2^40) */
static long long st_count(const st_tensor *t) {
    if (t->rank > 4) return -1;
    long long n = 1;
    for (int i = 0; i < t->rank; i++) {
        const long long d = t->shape[i];
        if (d < 0 || (d > 0 && n > (1LL << 40) / d)) return -1;
        n *= d;
    }
    return n;
}

/* bf16 tensor of exactly `elems` elements, straight out of the mapping */
static const uint16_t *st_bf16(const st_file *f, const char *name, long long elems) {
    const st_tensor *t = st_find(f, name);
    if (!t) return NULL;
    if (strcmp(t->dtype, "BF16") || st_count(t) != elems || t->end - t->begin != 2 * elems) {
        vt_set_error("safetensors: %s is not bf16 with %lld elements", name, elems);
        return NULL;
    }
    return (const uint16_t *)(f->map + f->data0 + t->begin);
}

/* f32 copy (caller frees) of a bf16, f16 or f32 tensor of `elems` elements */
static float *st_f32(const st_file *f, const char *name, long long elems) {
    const st_tensor *t = st_find(f, name);
    if (!t) return NULL;
    if (st_count(t) != elems) {                   /* present but of another size: an error, not "absent" */
        vt_set_error("safetensors: %s has %lld elements, expected %lld", name, st_count(t), elems);
        return NULL;
    }
    float *out = (float *)malloc(sizeof(float) * (size_t)elems);
    if (!out) return NULL;
    const unsigned char *src = f->map + f->data0 + t->begin;
    if (!strcmp(t->dtype, "F32") && t->end - t->begin == 4 * elems) {
        memcpy(out, src, sizeof(float) * (size_t)elems);
    } else if (!strcmp(t->dtype, "BF16") && t->end - t->begin == 2 * elems) {
        for (long long i = 0; i < elems; i++) {
            const unsigned bits = (unsigned)(src[2 * i] | (src[2 * i + 1] << 8)) << 16;
            memcpy(&out[i], &bits, 4);
        }
    } else if (!strcmp(t->dtype, "F16") && t->end - t->begin == 2 * elems) {
        for (long long i = 0; i < elems; i++) {
            const unsigned h = (unsigned)(src[2 * i] | (src[2 * i + 1] << 8));
            const int e = (int)((h >> 10) & 31), m = (int)(h & 1023);
            /* subnormals scale the mantissa alone; 31 is inf / nan */
            float v = e == 0 ? ldexpf((float)m, -24) : e == 31 ? (m ? NAN : INFINITY) : ldexpf((float)(m | 1024), e - 25);
            out[i] = (h & 0x8000) ? -v : v;
        }
    } else {
        vt_set_error("safetensors: %s is none of f32, f16, bf16", name);
        free(out);
        return NULL;
    }
    return out;
}

/* ---- C ABI ------------------------------------------------------------------------------ */

/* Looks one tensor up (no GPU involved): 0 and its dtype / rank / shape / byte size, 1 when the
 * file has no such tensor, -1 when the file cannot be read. */
/* The time-embedding frequencies a checkpoint without `time_embedding.inv_freq` gets:
 * f[i] = exp(-log(10000) i / half_dim) in fp32, operations in the order of
 * voxtral_tts_acoustic.c:48-60.  Host only. */
extern "C" void tts_hip_default_time_inv_freq(float *out, int half_dim) {
    const float theta = 10000.0f;
    for (int i = 0; i < half_dim; i++) out[i] = expf(-logf(theta) * (float)i / (float)half_dim);
}

extern "C" int tts_hip_safetensors_probe(const char *path, const char *name, char *dtype8, int *rank,
                                         long long *shape4, long long *nbytes) {
    st_file f;
    if (st_open(&f, path)) return -1;
    const st_tensor *t = st_find(&f, name);
    int rc = 1;
    if (t) {
        if (dtype8) { strncpy(dtype8, t->dtype, 7); dtype8[7] = 0; }
        if (rank) *rank = t->rank;
        if (shape4) for (int i = 0; i < 4; i++) shape4[i] = i < t->rank ? t->shape[i] : 0;
        if (nbytes) *nbytes = t->end - t->begin;
        rc = 0;
    }
    st_close(&f);
    return rc;
}

static int load_layer(const st_file *f, const char *prefix, int i, tts_hip_host_layer_t *l, float **norms) {
    char name[200];
#define VT_NAME(suffix) (snprintf(name, sizeof name, "%slayers.%d.%s", prefix, i, suffix), name)
    l->wq_bf16 = (uint16_t *)st_bf16(f, VT_NAME("attention.wq.weight"), (long long)VT_Q_DIM * VT_DIM);
    l->wk_bf16 = (uint16_t *)st_bf16(f, VT_NAME("attention.wk.weight"), (long long)VT_KV_DIM * VT_DIM);
    l->wv_bf16 = (uint16_t *)st_bf16(f, VT_NAME("attention.wv.weight"), (long long)VT_KV_DIM * VT_DIM);
    l->wo_bf16 = (uint16_t *)st_bf16(f, VT_NAME("attention.wo.weight"), (long long)VT_DIM * VT_Q_DIM);
    l->w1_bf16 = (uint16_t *)st_bf16(f, VT_NAME("feed_forward.w1.weight"), (long long)VT_FFN * VT_DIM);
    l->w2_bf16 = (uint16_t *)st_bf16(f, VT_NAME("feed_forward.w2.weight"), (long long)VT_DIM * VT_FFN);
    l->w3_bf16 = (uint16_t *)st_bf16(f, VT_NAME("feed_forward.w3.weight"), (long long)VT_FFN * VT_DIM);
    l->attention_norm = norms[0] = st_f32(f, VT_NAME("attention_norm.weight"), VT_DIM);
    l->ffn_norm = norms[1] = st_f32(f, VT_NAME("ffn_norm.weight"), VT_DIM);
#undef VT_NAME
    return l->wq_bf16 && l->wk_bf16 && l->wv_bf16 && l->wo_bf16 && l->w1_bf16 && l->w2_bf16 && l->w3_bf16 &&
           l->attention_norm && l->ffn_norm;
}

/* ---- codec decoder (tts_codec_load, voxtral_tts_codec.c:177-270) ---------------------------- */

struct st_pool { float *p[160]; int n; };
static float *st_keep(st_pool *pool, float *p) { if (p && pool->n < 160) pool->p[pool->n++] = p; return p; }

/* weight-normed convolution: effective weight = v * g / |v| per row (voxtral_tts_codec.c:38-57,
 * 71-119), or the plain .conv.weight of a checkpoint without the parametrisation */
static int load_conv(const st_file *f, st_pool *pool, const char *prefix, tts_hip_host_conv_t *cv, int in_ch,
                     int out_ch, int kernel, int stride, int transpose) {
    char name[256];
    const int rows = transpose ? in_ch : out_ch, fan_in = (transpose ? out_ch : in_ch) * kernel;
    const long long n = (long long)rows * fan_in;
    snprintf(name, sizeof name, "%s.conv.parametrizations.weight.original0", prefix);
    float *g = st_f32(f, name, rows);
    snprintf(name, sizeof name, "%s.conv.parametrizations.weight.original1", prefix);
    float *v = st_f32(f, name, n);
    if (g && v) {
        for (int o = 0; o < rows; o++) {
            float *row = v + (size_t)o * fan_in;
            float nsq = 0.0f;
            for (int i = 0; i < fan_in; i++) nsq += row[i] * row[i];
            const float scale = g[o] / sqrtf(nsq + 1e-12f);
            for (int i = 0; i < fan_in; i++) row[i] *= scale;
        }
        free(g);
        cv->weight = st_keep(pool, v);
    } else {
        free(g); free(v);
        snprintf(name, sizeof name, "%s.conv.weight", prefix);
        cv->weight = st_keep(pool, st_f32(f, name, n));
    }
    snprintf(name, sizeof name, "%s.conv.bias", prefix);
    cv->bias = st_keep(pool, st_f32(f, name, out_ch));
    cv->in_ch = in_ch; cv->out_ch = out_ch; cv->kernel = kernel; cv->stride = stride; cv->is_transpose = transpose;
    return cv->weight != NULL;
}

static int load_codec(const st_file *f, const char *path) {
    tts_hip_host_codec_t *c = (tts_hip_host_codec_t *)calloc(1, sizeof *c);
    st_pool pool;
    pool.n = 0;
    int ok = c != NULL, rc = -1;
    char name[256];
    if (ok) {
        float *sum = st_f32(f, "audio_tokenizer.quantizer.semantic_codebook.embedding_sum", 8192LL * 256);
        float *usage = st_f32(f, "audio_tokenizer.quantizer.semantic_codebook.cluster_usage", 8192);
        ok = sum && usage;
        for (int i = 0; ok && i < 8192; i++) {
            const float u = usage[i] < 1e-5f ? 1e-5f : usage[i];
            for (int j = 0; j < 256; j++) sum[i * 256 + j] /= u;
        }
        free(usage);
        c->semantic_embedding = st_keep(&pool, sum);
        for (int h = 0; h < 8; h++) c->alibi_slopes[h] = powf(2.0f, -8.0f / 8.0f * (float)(h + 1));
    }
    ok = ok && load_conv(f, &pool, "audio_tokenizer.decoder_blocks.0", &c->input_conv, 292, 1024, 3, 1, 0);
    static const int windows[4] = {2, 4, 8, 16};
    int block = 1;
    for (int stage = 0; ok && stage < 4; stage++) {
        for (int l = 0; ok && l < 2; l++) {
            tts_hip_host_codec_layer_t *L = &c->transformers[stage * 2 + l];
#define VT_CT(field, suffix, count) \
            (snprintf(name, sizeof name, "audio_tokenizer.decoder_blocks.%d.layers.%d." suffix, block, l), \
             L->field = st_keep(&pool, st_f32(f, name, count)))
            VT_CT(wq, "attention.wq.weight", 1024LL * 1024); VT_CT(wk, "attention.wk.weight", 1024LL * 1024);
            VT_CT(wv, "attention.wv.weight", 1024LL * 1024); VT_CT(wo, "attention.wo.weight", 1024LL * 1024);
            VT_CT(q_norm, "attention.q_norm.weight", 1024); VT_CT(k_norm, "attention.k_norm.weight", 1024);
            VT_CT(attention_norm, "attention_norm.weight", 1024); VT_CT(ffn_norm, "ffn_norm.weight", 1024);
            VT_CT(w1, "feed_forward.w1.weight", 4096LL * 1024); VT_CT(w2, "feed_forward.w2.weight", 1024LL * 4096);
            VT_CT(w3, "feed_forward.w3.weight", 4096LL * 1024);
            VT_CT(attn_scale, "attention_scale", 1024); VT_CT(ffn_scale, "ffn_scale", 1024);
#undef VT_CT
            L->window_size = windows[stage];
            ok = L->wq && L->wk && L->wv && L->wo && L->attention_norm && L->ffn_norm && L->w1 && L->w2 && L->w3;
        }
        block++;
        if (ok && stage < 3) {
            snprintf(name, sizeof name, "audio_tokenizer.decoder_blocks.%d", block);
            ok = load_conv(f, &pool, name, &c->stage_convs[stage], 1024, 1024, 4, 2, 1);
            block++;
        }
    }
    ok = ok && load_conv(f, &pool, "audio_tokenizer.output_proj", &c->output_proj, 1024, 240, 7, 1, 0);
    if (!ok) vt_set_error("safetensors: codec decoder of %s is incomplete", path);
    else rc = tts_hip_upload_codec_weights(c);
    for (int i = 0; i < pool.n; i++) free(pool.p[i]);
    free(c);
    return rc;
}

/* Uploads what the file holds under the reference's tensor names: backbone layers 0..n-1 (as
 * many consecutive ones as are present, at most 26) with norm.weight, the acoustic
 * transformer (all of it or none), the audio-code embedding table, the codec decoder.  Returns a
 * bit mask (1 backbone, 2 acoustic, 4 audio embeddings, 8 codec decoder; the number of backbone layers is in
 * g_hip.dec_layers_uploaded) or -1.  tts_hip_init must have been called. */
extern "C" int tts_hip_load_safetensors(const char *path) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_load_safetensors: backend not initialised"); return -1; }
    st_file f;
    if (st_open(&f, path)) return -1;
    int mask = 0, rc = 0;
    const int errs_at_start = g_vt.error_count;
    float *tofree[2 * (TTS_HIP_DEC_LAYERS + TTS_HIP_AC_LAYERS) + 8];
    int nfree = 0;

    /* backbone */
    {
        tts_hip_host_decoder_t *dec = (tts_hip_host_decoder_t *)calloc(1, sizeof *dec);
        int n = 0;
        if (dec && st_find(&f, "layers.0.attention.wq.weight")) {
            const int errs0 = g_vt.error_count;
            for (; n < TTS_HIP_DEC_LAYERS; n++) {
                char probe[64];
                snprintf(probe, sizeof probe, "layers.%d.attention.wq.weight", n);
                if (!st_find(&f, probe)) break;
                if (!load_layer(&f, "", n, &dec->layers[n], &tofree[nfree])) { rc = -1; break; }
                nfree += 2;
            }
            dec->norm = tofree[nfree++] = st_f32(&f, "norm.weight", VT_DIM);
            if (st_find(&f, "mm_audio_embeddings.tok_embeddings.weight"))
                dec->tok_embeddings_bf16 = (uint16_t *)st_bf16(&f, "mm_audio_embeddings.tok_embeddings.weight", 131072LL * VT_DIM);
            if (!rc && (!dec->norm || g_vt.error_count != errs0)) rc = -1;
            if (rc) vt_set_error("safetensors: backbone layer %d of %s is incomplete", n, path);
            if (!rc && n > 0 && tts_hip_upload_llm_weights_n(dec, n) == 0) mask |= 1;
            else if (!rc && n > 0) rc = -1;
        }
        free(dec);
    }
    /* acoustic transformer */
    if (!rc && st_find(&f, "acoustic_transformer.input_projection.weight")) {
        tts_hip_host_acoustic_t *ac = (tts_hip_host_acoustic_t *)calloc(1, sizeof *ac);
        int ok = ac != NULL;
        if (ok) {
            ac->time_inv_freq = tofree[nfree++] = st_f32(&f, "acoustic_transformer.time_embedding.inv_freq", VT_DIM / 2);
            if (!ac->time_inv_freq) {
                /* not in the checkpoint: the closed form of voxtral_tts_acoustic.c:48-60 */
                float *tf = (float *)malloc(sizeof(float) * (VT_DIM / 2));
                ok = tf != NULL;
                if (ok) tts_hip_default_time_inv_freq(tf, VT_DIM / 2);
                ac->time_inv_freq = tofree[nfree - 1] = tf;
            }
            ac->input_proj_bf16 = (uint16_t *)st_bf16(&f, "acoustic_transformer.input_projection.weight", (long long)VT_DIM * VT_AC_DIM_IN);
            ac->time_proj_bf16 = (uint16_t *)st_bf16(&f, "acoustic_transformer.time_projection.weight", (long long)VT_DIM * VT_DIM);
            ac->llm_proj_bf16 = (uint16_t *)st_bf16(&f, "acoustic_transformer.llm_projection.weight", (long long)VT_DIM * VT_DIM);
            ac->semantic_out_bf16 = (uint16_t *)st_bf16(&f, "acoustic_transformer.semantic_codebook_output.weight", (long long)VT_SEM_PADDED * VT_DIM);
            ac->acoustic_out_bf16 = (uint16_t *)st_bf16(&f, "acoustic_transformer.acoustic_codebook_output.weight", (long long)VT_AC_DIM_IN * VT_DIM);
            ac->semantic_out_bias = tofree[nfree++] = st_f32(&f, "acoustic_transformer.semantic_codebook_output.bias", VT_SEM_PADDED);
            ac->norm = tofree[nfree++] = st_f32(&f, "acoustic_transformer.norm.weight", VT_DIM);
            ok = ok && ac->input_proj_bf16 && ac->time_proj_bf16 && ac->llm_proj_bf16 && ac->semantic_out_bf16 &&
                 ac->acoustic_out_bf16 && ac->norm;
            for (int i = 0; ok && i < TTS_HIP_AC_LAYERS; i++) {
                ok = load_layer(&f, "acoustic_transformer.", i, &ac->layers[i], &tofree[nfree]);
                nfree += 2;
            }
        }
        if (!ok) { vt_set_error("safetensors: acoustic transformer of %s is incomplete", path); rc = -1; }
        else if (tts_hip_upload_acoustic_weights(ac) == 0) mask |= 2;
        else rc = -1;
        free(ac);
    }
    /* audio-code embeddings: codebook offsets as in voxtral_tts_voice.c:268-284 */
    if (!rc) {
        const st_tensor *t = st_find(&f, "mm_audio_embeddings.audio_codebook_embeddings.embeddings.weight");
        if (t) {
            const long long rows = t->rank == 2 && t->shape[1] == VT_DIM ? t->shape[0] : -1;
            const uint16_t *emb = rows > 0 ? st_bf16(&f, t->name, rows * VT_DIM) : NULL;
            int offs[1 + VT_AC_DIM_IN];
            offs[0] = 0;
            offs[1] = 8192 + 2;
            for (int i = 2; i <= VT_AC_DIM_IN; i++) offs[i] = offs[i - 1] + 21 + 2;
            if (!emb || rows < offs[VT_AC_DIM_IN] + 23) { vt_set_error("safetensors: audio embedding table of %s has a wrong shape", path); rc = -1; }
            else if (tts_hip_upload_audio_embeddings(emb, (int)rows, offs) == 0) mask |= 4;
            else rc = -1;
        }
    }
    if (!rc && st_find(&f, "audio_tokenizer.quantizer.semantic_codebook.embedding_sum")) {
        if (load_codec(&f, path) == 0) mask |= 8;
        else rc = -1;
    }
    for (int i = 0; i < nfree; i++) free(tofree[i]);
    st_close(&f);
    /* a tensor that is present under a known name but has the wrong size or type fails the load,
     * also where the tensor is optional */
    if (!rc && g_vt.error_count != errs_at_start) rc = -1;
    return rc ? -1 : mask;
}
