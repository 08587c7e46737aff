/* model_folder.c - see model_folder.h.  The reader works on one table of every shard's entries sorted by name: a logical
 * tensor is recognised from one entry (X.seeds, X.scales, X.tcq_words, or a BF16 entry) and its other streams are looked
 * up by name, as the reference's ns_open does (nslm/lib_model_st.c:158-279).  C99 + POSIX. */
#define _POSIX_C_SOURCE 200809L
#include "model_folder.h"

#include <dirent.h>
#include <errno.h>
#include <fcntl.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include "nslm_rt.h"

/* ---------------------------------------------------------------------------------------------------------------------
 * A JSON cursor: strict enough that a truncated or malformed document is an error, never a read past the buffer. */
typedef struct {
    const char* p;
    const char* e;
} Jc;

static void jc_ws(Jc* j) {
    while (j->p < j->e && (*j->p == ' ' || *j->p == '\n' || *j->p == '\r' || *j->p == '\t')) ++j->p;
}
static int jc_eat(Jc* j, char c) {
    jc_ws(j);
    if (j->p < j->e && *j->p == c) { ++j->p; return 1; }
    return 0;
}
static int jc_peek(Jc* j) {
    jc_ws(j);
    return j->p < j->e ? (unsigned char) *j->p : -1;
}
/* A string into out (cap bytes, truncated, NUL-terminated; out may be NULL).  \uXXXX below 0x80 is decoded, others kept
 * as '?': names here are ASCII.  1, or 0 on malformed input. */
static int jc_string(Jc* j, char* out, size_t cap) {
    size_t n = 0;
    if (!jc_eat(j, '"')) return 0;
    while (j->p < j->e && *j->p != '"') {
        char c = *j->p++;
        if (c == '\\') {
            if (j->p >= j->e) return 0;
            const char x = *j->p++;
            switch (x) {
            case 'n': c = '\n'; break;
            case 't': c = '\t'; break;
            case 'r': c = '\r'; break;
            case 'b': c = '\b'; break;
            case 'f': c = '\f'; break;
            case 'u': {
                if (j->e - j->p < 4) return 0;
                unsigned v = 0;
                for (int i = 0; i < 4; ++i) {
                    const char h = j->p[i];
                    const int d = h >= '0' && h <= '9' ? h - '0' : h >= 'a' && h <= 'f' ? h - 'a' + 10 : h >= 'A' && h <= 'F' ? h - 'A' + 10 : -1;
                    if (d < 0) return 0;
                    v = v * 16 + (unsigned) d;
                }
                j->p += 4;
                c = v < 0x80 ? (char) v : '?';
                break;
            }
            default: c = x;   /* \" \\ \/ */
            }
        }
        if (out && n + 1 < cap) out[n++] = c;
    }
    if (out && cap) out[n] = 0;
    if (j->p >= j->e) return 0;
    ++j->p;
    return 1;
}
/* A non-negative integer that fits 63 bits (shapes, offsets, bits, group sizes).  1, or 0 (negative, fraction, overflow). */
static int jc_uint(Jc* j, uint64_t* v) {
    jc_ws(j);
    const char* s = j->p;
    uint64_t x = 0;
    while (j->p < j->e && *j->p >= '0' && *j->p <= '9') {
        const uint64_t d = (uint64_t) (*j->p - '0');
        if (x > (UINT64_MAX - d) / 10) return 0;
        x = x * 10 + d;
        ++j->p;
    }
    if (j->p == s || (j->p < j->e && (*j->p == '.' || *j->p == 'e' || *j->p == 'E'))) return 0;
    *v = x;
    return 1;
}
static int jc_skip(Jc* j, int depth);
static int jc_literal(Jc* j, const char* w) {
    const size_t n = strlen(w);
    if ((size_t) (j->e - j->p) < n || memcmp(j->p, w, n)) return 0;
    j->p += n;
    return 1;
}
/* Any value.  1, or 0 on malformed or truncated input. */
static int jc_skip(Jc* j, int depth) {
    if (depth > 64) return 0;
    const int c = jc_peek(j);
    if (c == '"') return jc_string(j, NULL, 0);
    if (c == '{' || c == '[') {
        const char close = c == '{' ? '}' : ']';
        ++j->p;
        if (jc_eat(j, close)) return 1;
        do {
            if (c == '{' && (!jc_string(j, NULL, 0) || !jc_eat(j, ':'))) return 0;
            if (!jc_skip(j, depth + 1)) return 0;
        } while (jc_eat(j, ','));
        return jc_eat(j, close);
    }
    if (c == 't') return jc_literal(j, "true");
    if (c == 'f') return jc_literal(j, "false");
    if (c == 'n') return jc_literal(j, "null");
    if (c == '-' || (c >= '0' && c <= '9')) {
        const char* s = j->p;
        if (*j->p == '-') ++j->p;
        while (j->p < j->e && ((*j->p >= '0' && *j->p <= '9') || *j->p == '.' || *j->p == 'e' || *j->p == 'E' || *j->p == '+' || *j->p == '-')) ++j->p;
        return j->p > s + (*s == '-');
    }
    return 0;
}
/* Inside an object whose '{' is consumed: position the cursor at the value of member `key`.  1 found, 0 absent (cursor
 * after '}'), -1 malformed. */
static int jc_member(Jc* j, const char* key) {
    if (jc_eat(j, '}')) return 0;
    do {
        char k[176];
        if (!jc_string(j, k, sizeof k) || !jc_eat(j, ':')) return -1;
        if (!strcmp(k, key)) return 1;
        if (!jc_skip(j, 0)) return -1;
    } while (jc_eat(j, ','));
    return jc_eat(j, '}') ? 0 : -1;
}
/* The object value of path a(.b) from the document's top: cursor just after its '{'.  1, 0 absent, -1 malformed. */
static int jc_object_at(Jc* j, const char* doc, size_t n, const char* a, const char* b) {
    j->p = doc;
    j->e = doc + n;
    if (!jc_eat(j, '{')) return -1;
    int r = jc_member(j, a);
    if (r != 1) return r;
    if (!jc_eat(j, '{')) return 0;
    if (!b) return 1;
    r = jc_member(j, b);
    if (r != 1) return r;
    return jc_eat(j, '{') ? 1 : 0;
}

/* ---------------------------------------------------------------------------------------------------------------------
 * Shards */
typedef struct {
    char name[96];
    char dtype[8];
    int ndim, shard;
    int64_t shape[8];
    uint64_t begin, end; /* relative to the shard's data section */
} Entry;

typedef struct {
    const uint8_t* map;
    size_t size;
    uint64_t data; /* file offset of the data section */
} Shard;

struct NsfModel {
    Shard* sh;
    int nsh;
    Entry* e;
    int ne;
    NsfTensor* t;
    int n;
};

static int fail(char* err, int errlen, const char* fmt, const char* a, const char* b) {
    if (err && errlen > 0) snprintf(err, (size_t) errlen, fmt, a, b);
    return -1;
}

static uint64_t row_words_tcq(int cols, int T, int L, int K) { /* nslm/trellis.h:30-35 */
    const uint64_t bits = (uint64_t) ((cols + T - 1) / T) * ((uint64_t) K * (uint64_t) T + (uint64_t) (L - K));
    return (bits + 31) / 32 + 1;
}
static uint64_t stream_len(int enc, int slices, int rows, int cols, int group, int s) { /* nslm/lib_model_st.c:36-60 */
    const uint64_t n = (uint64_t) slices * (uint64_t) rows * (uint64_t) cols;
    if (s < 0 || s > 3) return 0;
    switch (enc) {
    case NSF_BF16: return s == 0 ? 2 * n : 0;
    case NSF_Q8: return s == 0 ? n : s < 3 ? 2 * (n / (uint64_t) group) : 0;
    case NSF_Q4: return s == 0 ? n / 2 : s < 3 ? 2 * (n / (uint64_t) group) : 0;
    case NSF_SEED4: return s < 2 ? 2 * (n / 8) : s == 2 ? 4 * (uint64_t) slices : 0;
    case NSF_SEED4P4: return s < 2 ? 2 * (n / 8) : s == 2 ? 4 * (uint64_t) slices : n / 16;
    case NSF_SEED6P8: return s == 0 ? 2 * (n / 8) : s == 1 ? 4 * (n / 8) : s == 2 ? 4 * (uint64_t) slices : n / 16;
    case NSF_TCQ: {
        const int L = group & 255, K = group >> 8 & 255, T = group >> 16;
        if (T < 1 || K < 1 || K >= L || L > 16) return 0;
        const uint64_t sr = (uint64_t) slices * (uint64_t) rows;
        return s == 0 ? 4 * sr * row_words_tcq(cols, T, L, K) : s == 1 ? 2 * sr * (uint64_t) ((cols + T - 1) / T) : 0;
    }
    default: return 0;
    }
}
uint64_t nsf_stream_len(int enc, int slices, int rows, int cols, int s) { return stream_len(enc, slices, rows, cols, 64, s); }

static int ends_with(const char* s, const char* suf) {
    const size_t a = strlen(s), b = strlen(suf);
    return a >= b && !strcmp(s + a - b, suf);
}

/* The header of one mapped shard into m->e.  0, or -1 (malformed). */
static int parse_header(NsfModel* m, int shard, const char* hdr, size_t hn, int* cap) {
    Jc j = {hdr, hdr + hn};
    if (!jc_eat(&j, '{')) return -1;
    if (jc_eat(&j, '}')) return 0;
    do {
        char key[176];
        if (!jc_string(&j, key, sizeof key) || !jc_eat(&j, ':')) return -1;
        if (!strcmp(key, "__metadata__")) {
            if (!jc_skip(&j, 0)) return -1;
            continue;
        }
        if (strlen(key) >= sizeof m->e[0].name) return -1;
        if (m->ne == *cap) {
            *cap = *cap ? 2 * *cap : 256;
            m->e = (Entry*) realloc(m->e, sizeof(Entry) * (size_t) *cap);
        }
        Entry* t = &m->e[m->ne];
        memset(t, 0, sizeof *t);
        memcpy(t->name, key, strlen(key) + 1);
        t->shard = shard;
        int have_off = 0;
        if (!jc_eat(&j, '{')) return -1;
        if (!jc_eat(&j, '}')) {
            do {
                char f[32];
                if (!jc_string(&j, f, sizeof f) || !jc_eat(&j, ':')) return -1;
                if (!strcmp(f, "dtype")) {
                    if (!jc_string(&j, t->dtype, sizeof t->dtype)) return -1;
                } else if (!strcmp(f, "shape") || !strcmp(f, "data_offsets")) {
                    uint64_t v[8];
                    int k = 0;
                    if (!jc_eat(&j, '[')) return -1;
                    if (!jc_eat(&j, ']')) {
                        do {
                            if (k >= 8 || !jc_uint(&j, &v[k])) return -1;   /* negative, fractional or huge: refused */
                            ++k;
                        } while (jc_eat(&j, ','));
                        if (!jc_eat(&j, ']')) return -1;
                    }
                    if (f[0] == 's') {
                        t->ndim = k;
                        for (int i = 0; i < k; ++i) {
                            if (v[i] > (uint64_t) INT64_MAX) return -1;
                            t->shape[i] = (int64_t) v[i];
                        }
                    } else {
                        if (k != 2) return -1;
                        t->begin = v[0];
                        t->end = v[1];
                        have_off = 1;
                    }
                } else if (!jc_skip(&j, 0)) return -1;
            } while (jc_eat(&j, ','));
            if (!jc_eat(&j, '}')) return -1;
        }
        if (!have_off || !t->dtype[0]) return -1;
        ++m->ne;
    } while (jc_eat(&j, ','));
    if (!jc_eat(&j, '}')) return -1;
    jc_ws(&j);
    return j.p == j.e ? 0 : -1;
}

static int open_shard(NsfModel* m, const char* path, int* cap, char* err, int errlen) {
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return fail(err, errlen, "%s: %s", path, strerror(errno));
    struct stat sb;
    if (fstat(fd, &sb) || sb.st_size < 8) {
        close(fd);
        return fail(err, errlen, "%s: not a safetensors file (%s)", path, "shorter than its header length");
    }
    void* map = mmap(NULL, (size_t) sb.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED) return fail(err, errlen, "%s: mmap failed (%s)", path, strerror(errno));
    m->sh = (Shard*) realloc(m->sh, sizeof(Shard) * (size_t) (m->nsh + 1));
    Shard* s = &m->sh[m->nsh++];
    s->map = (const uint8_t*) map;
    s->size = (size_t) sb.st_size;
    uint64_t hn;
    memcpy(&hn, s->map, 8);
    if (hn > s->size - 8 || hn > (100u << 20))   /* the format's limit: 100 MB of header (nslm/lib_format.c:66) */
        return fail(err, errlen, "%s: not a safetensors file (%s)", path, "header longer than the file");
    s->data = 8 + hn;
    const int first = m->ne;
    if (parse_header(m, m->nsh - 1, (const char*) s->map + 8, (size_t) hn, cap))
        return fail(err, errlen, "%s: cannot parse the safetensors header%s", path, "");
    for (int i = first; i < m->ne; ++i)
        if (m->e[i].begin > m->e[i].end || m->e[i].end > s->size - s->data) return fail(err, errlen, "%s: %s is out of bounds", path, m->e[i].name);
    return 0;
}

static char* slurp(const char* dir, const char* name, size_t* n) {
    char path[2048];
    snprintf(path, sizeof path, "%s/%s", dir, name);
    FILE* f = fopen(path, "rb");
    if (!f) return NULL;
    char* s = NULL;
    long len = -1;
    if (!fseek(f, 0, SEEK_END) && (len = ftell(f)) >= 0 && !fseek(f, 0, SEEK_SET) && (s = (char*) malloc((size_t) len + 1))) {
        *n = fread(s, 1, (size_t) len, f);
        s[*n] = 0;
    }
    fclose(f);
    return s;
}

static int str_cmp(const void* a, const void* b) { return strcmp(*(char* const*) a, *(char* const*) b); }
static int entry_cmp(const void* a, const void* b) { return strcmp(((const Entry*) a)->name, ((const Entry*) b)->name); }
static int tensor_cmp(const void* a, const void* b) { return strcmp(((const NsfTensor*) a)->name, ((const NsfTensor*) b)->name); }

/* Shard file names: the distinct values of the index's weight_map, else model*.safetensors of the folder; sorted. */
static int shard_names(const char* dir, char*** out, char* err, int errlen) {
    char** v = NULL;
    int n = 0;
    size_t len = 0;
    char* idx = slurp(dir, "model.safetensors.index.json", &len);
    if (idx) {
        Jc j;
        const int r = jc_object_at(&j, idx, len, "weight_map", NULL);
        if (r != 1) {
            free(idx);
            return fail(err, errlen, "%s/model.safetensors.index.json: no weight_map%s", dir, "");
        }
        int bad = 0;
        if (!jc_eat(&j, '}')) {
            do {
                char file[512];
                if (!jc_string(&j, NULL, 0) || !jc_eat(&j, ':')) { bad = 1; break; }
                if (jc_peek(&j) != '"') {
                    if (!jc_skip(&j, 0)) { bad = 1; break; }
                    continue;
                }
                if (!jc_string(&j, file, sizeof file)) { bad = 1; break; }
                if (strchr(file, '/')) continue;
                int seen = 0;
                for (int k = 0; k < n && !seen; ++k) seen = !strcmp(v[k], file);
                if (seen) continue;
                v = (char**) realloc(v, sizeof(char*) * (size_t) (n + 1));
                v[n++] = strdup(file);
            } while (jc_eat(&j, ','));
            if (!bad && !jc_eat(&j, '}')) bad = 1;
        }
        free(idx);
        if (bad) {
            for (int i = 0; i < n; ++i) free(v[i]);
            free(v);
            return fail(err, errlen, "%s/model.safetensors.index.json: cannot parse%s", dir, "");
        }
    } else {
        DIR* d = opendir(dir);
        if (!d) return fail(err, errlen, "%s: %s", dir, strerror(errno));
        for (struct dirent* de; (de = readdir(d));)
            if (!strncmp(de->d_name, "model", 5) && ends_with(de->d_name, ".safetensors")) {
                v = (char**) realloc(v, sizeof(char*) * (size_t) (n + 1));
                v[n++] = strdup(de->d_name);
            }
        closedir(d);
    }
    if (!n) {
        free(v);
        return fail(err, errlen, "%s: no safetensors%s", dir, "");
    }
    qsort(v, (size_t) n, sizeof(char*), str_cmp);
    *out = v;
    return n;
}

static const Entry* lookup(const NsfModel* m, const char* name) {
    Entry k;
    if (strlen(name) >= sizeof k.name) return NULL;
    snprintf(k.name, sizeof k.name, "%s", name);
    return m->ne ? (const Entry*) bsearch(&k, m->e, (size_t) m->ne, sizeof(Entry), entry_cmp) : NULL;
}

/* [slices,] rows, cols of an entry (nslm/lib_model_st.c:127-140): 3-D, 2-D, or (unless the last dimension must be a
 * packed one) 1-D.  0, -1 not a weight shape, -2 out of range (each dimension an int, the tensor at most 2^40 values). */
static int dims(const Entry* e, int want_last, int64_t* s, int64_t* r, int64_t* c) {
    if (e->ndim == 3) { *s = e->shape[0]; *r = e->shape[1]; *c = e->shape[2]; }
    else if (e->ndim == 2) { *s = 1; *r = e->shape[0]; *c = e->shape[1]; }
    else if (e->ndim == 1 && !want_last) { *s = 1; *r = 1; *c = e->shape[0]; }
    else return -1;
    const int64_t lim = (int64_t) 1 << 40;
    if (*s < 1 || *r < 1 || *c < 1 || *s > INT32_MAX / 16 || *r > INT32_MAX / 16 || *c > INT32_MAX / 64) return -2;
    return *s * *r > lim || *s * *r * *c > lim ? -2 : 0;
}

static const char* SUFFIX[9][4] = {
    [NSF_BF16] = {"", NULL, NULL, NULL},
    [NSF_SEED4] = {".seeds", ".nibbles", ".exp_bias", NULL},
    [NSF_Q8] = {".weight", ".scales", ".biases", NULL},
    [NSF_Q4] = {".weight", ".scales", ".biases", NULL},
    [NSF_SEED4P4] = {".seeds", ".coefs", ".exp_bias", ".codes"},
    [NSF_SEED6P8] = {".seeds", ".coefs", ".exp_bias", ".codes"},
    [NSF_TCQ] = {".tcq_words", ".tcq_scales", NULL, NULL},
};
static const char* DTYPE[9][4] = {
    [NSF_BF16] = {"BF16", NULL, NULL, NULL},
    [NSF_SEED4] = {"U16", "U16", "I32", NULL},
    [NSF_Q8] = {"U32", "BF16", "BF16", NULL},
    [NSF_Q4] = {"U32", "BF16", "BF16", NULL},
    [NSF_SEED4P4] = {"U16", "U16", "I32", "U8"},
    [NSF_SEED6P8] = {"U16", "U32", "I32", "U8"},
    [NSF_TCQ] = {"U32", "BF16", NULL, NULL},
};

static int add_tensor(NsfModel* m, int* cap, const char* base, const char* name, int enc, int group, int64_t S, int64_t R, int64_t C,
                      char* err, int errlen) {
    NsfTensor t;
    memset(&t, 0, sizeof t);
    if (strlen(name) >= sizeof t.name) return fail(err, errlen, "%s: name too long%s", name, "");
    snprintf(t.name, sizeof t.name, "%s", name);
    t.enc = enc; t.slices = (int) S; t.rows = (int) R; t.cols = (int) C; t.group = group;
    for (int s = 0; s < 4 && SUFFIX[enc][s]; ++s) {
        char nm[200];
        const int bare = !s && !strcmp(name, base);   /* an affine tensor not named *.weight: its codes are named X */
        snprintf(nm, sizeof nm, "%s%s", base, bare ? "" : SUFFIX[enc][s]);
        const Entry* e = lookup(m, nm);
        const uint64_t want = stream_len(enc, t.slices, t.rows, t.cols, group, s);
        if (!e || strcmp(e->dtype, DTYPE[enc][s]) || e->end - e->begin != want) {
            char what[64];
            snprintf(what, sizeof what, "%s with %llu bytes", DTYPE[enc][s], (unsigned long long) want);
            return fail(err, errlen, "%s: missing, or not %s", nm, what);
        }
        const Shard* f = &m->sh[e->shard];
        t.s[s].p = f->map + f->data + e->begin;
        t.s[s].len = want;
        t.s[s].off = f->data + e->begin;
        t.s[s].shard = e->shard;
    }
    if (m->n == *cap) {
        *cap = *cap ? 2 * *cap : 64;
        m->t = (NsfTensor*) realloc(m->t, sizeof(NsfTensor) * (size_t) *cap);
    }
    m->t[m->n++] = t;
    return 0;
}

/* bits and group_size of config.json's quantization entry for module `base` (MLX: top level "quantization" or
 * "quantization_config", or text_config.quantization; nslm/lib_model_st.c:176-179,243-246).  Zero when absent. */
static void module_quant(const char* cfg, size_t n, const char* base, uint64_t* bits, uint64_t* group) {
    static const char* where[3][2] = {{"quantization", NULL}, {"quantization_config", NULL}, {"text_config", "quantization"}};
    *bits = *group = 0;
    if (!cfg) return;
    for (int w = 0; w < 3; ++w) {
        Jc j;
        if (jc_object_at(&j, cfg, n, where[w][0], where[w][1]) != 1) continue;
        if (jc_member(&j, base) != 1 || !jc_eat(&j, '{') || jc_eat(&j, '}')) return;
        do {
            char k[32];
            uint64_t v;
            if (!jc_string(&j, k, sizeof k) || !jc_eat(&j, ':')) return;
            const int c = jc_peek(&j);
            if ((!strcmp(k, "bits") || !strcmp(k, "group_size")) && c >= '0' && c <= '9' && jc_uint(&j, &v)) {
                if (k[0] == 'b') *bits = v;
                else *group = v;
            } else if (!jc_skip(&j, 0)) return;
        } while (jc_eat(&j, ','));
        return;
    }
}

NsfModel* nsf_open(const char* dir, char* err, int errlen) {
    char** names = NULL;
    if (err && errlen > 0) err[0] = 0;
    const int ns = shard_names(dir, &names, err, errlen);
    if (ns < 0) return NULL;
    NsfModel* m = (NsfModel*) calloc(1, sizeof *m);
    int ecap = 0, tcap = 0, rc = -1;
    size_t cfgn = 0;
    char* cfg = slurp(dir, "config.json", &cfgn);
    for (int i = 0; i < ns; ++i) {
        char path[2048];
        snprintf(path, sizeof path, "%s/%s", dir, names[i]);
        if (open_shard(m, path, &ecap, err, errlen)) goto done;
    }
    if (m->ne) qsort(m->e, (size_t) m->ne, sizeof(Entry), entry_cmp);
    for (int i = 1; i < m->ne; ++i)
        if (!strcmp(m->e[i].name, m->e[i - 1].name)) { fail(err, errlen, "%s appears twice%s", m->e[i].name, ""); goto done; }
    for (int i = 0; i < m->ne; ++i) {
        const Entry* e = &m->e[i];
        const char* nm = e->name;
        const size_t L = strlen(nm);
        char base[176], logical[200], k[200];
        int64_t S, R, C;
        if (ends_with(nm, ".tcq_words")) {   /* trellis rows: X.tcq_params holds L, K, T and cols */
            snprintf(base, sizeof base, "%.*s", (int) (L - 10), nm);
            snprintf(logical, sizeof logical, "%s.weight", base);
            snprintf(k, sizeof k, "%s.tcq_params", base);
            const Entry* pr = lookup(m, k);
            int32_t pv[4] = {0, 0, 0, 0};
            if (pr && !strcmp(pr->dtype, "I32") && pr->end - pr->begin == sizeof pv) memcpy(pv, m->sh[pr->shard].map + m->sh[pr->shard].data + pr->begin, sizeof pv);
            if (!pr || pv[2] < 1 || pv[1] < 1 || pv[1] >= pv[0] || pv[0] > 16 || pv[2] > 65535 || pv[3] < 1 || e->ndim != 3 || dims(e, 1, &S, &R, &C) ||
                (uint64_t) C != row_words_tcq(pv[3], pv[2], pv[0], pv[1])) {
                fail(err, errlen, "%s: not a trellis tensor (I32 L, K, T, cols in %s, U32 [E, rows, words])", nm, k);
                goto done;
            }
            if (add_tensor(m, &tcap, base, logical, NSF_TCQ, pv[0] | pv[1] << 8 | pv[2] << 16, S, R, pv[3], err, errlen)) goto done;
        } else if (ends_with(nm, ".seeds") || ends_with(nm, ".scales")) {
            const int seeds = ends_with(nm, ".seeds");
            snprintf(base, sizeof base, "%.*s", (int) (L - (seeds ? 6 : 7)), nm);
            snprintf(logical, sizeof logical, "%s.weight", base);
            if (dims(e, 1, &S, &R, &C)) { fail(err, errlen, "%s: bad shape%s", nm, ""); goto done; }
            int enc, group = 0;
            if (seeds) {   /* no .codes: P = 3; .coefs as U32: P = 8; else P = 4 */
                snprintf(k, sizeof k, "%s.coefs", base);
                const Entry* cf = lookup(m, k);
                snprintf(k, sizeof k, "%s.codes", base);
                enc = !lookup(m, k) ? NSF_SEED4 : cf && !strcmp(cf->dtype, "U32") ? NSF_SEED6P8 : NSF_SEED4P4;
                C *= 8;
            } else {
                /* bits x group = 32 x (code words a row) / (groups a row): 128 is Q4 g32, 256 Q4 g64 or Q8 g32, 512 Q8 g64;
                 * config.json's entry for the module, if any, tells Q4 g64 from Q8 g32 and must agree with the shapes */
                snprintf(k, sizeof k, "%s.weight", base);
                const Entry* w = lookup(m, k);
                if (!w && (w = lookup(m, base))) snprintf(logical, sizeof logical, "%s", base);
                const int64_t bg = w && w->ndim >= 1 && C ? w->shape[w->ndim - 1] * 32 / C : 0;
                uint64_t b, gs;
                module_quant(cfg, cfgn, base, &b, &gs);
                if (b ? (b != 4 && b != 8) || (gs != 32 && gs != 64) || (int64_t) (b * gs) != bg : bg != 128 && bg != 256 && bg != 512) {
                    fail(err, errlen, "%s: not affine Q4 or Q8 with group 32 or 64%s", base, "");
                    goto done;
                }
                enc = (b ? b == 8 : bg == 512) ? NSF_Q8 : NSF_Q4;
                group = b ? (int) gs : bg == 128 ? 32 : 64;
                C *= group;
            }
            if (add_tensor(m, &tcap, base, logical, enc, group, S, R, C, err, errlen)) goto done;
        } else if (!strcmp(e->dtype, "BF16")) {
            if (ends_with(nm, ".tcq_scales")) continue;
            if (ends_with(nm, ".biases")) {   /* a quantized tensor's biases */
                snprintf(k, sizeof k, "%.*s.scales", (int) (L - 7), nm);
                if (lookup(m, k)) continue;
            }
            const int d = dims(e, 0, &S, &R, &C);
            if (d == -1) continue;   /* scalars and > 3-D tensors are not model weights here */
            if (d) { fail(err, errlen, "%s: bad shape%s", nm, ""); goto done; }
            if (add_tensor(m, &tcap, nm, nm, NSF_BF16, 0, S, R, C, err, errlen)) goto done;
        }
    }
    if (m->n) qsort(m->t, (size_t) m->n, sizeof(NsfTensor), tensor_cmp);
    rc = 0;
done:
    free(cfg);
    for (int i = 0; i < ns; ++i) free(names[i]);
    free(names);
    if (rc) {
        nsf_close(m);
        return NULL;
    }
    return m;
}

void nsf_close(NsfModel* m) {
    if (!m) return;
    for (int i = 0; i < m->nsh; ++i) munmap((void*) m->sh[i].map, m->sh[i].size);
    free(m->sh);
    free(m->e);
    free(m->t);
    free(m);
}
int nsf_count(const NsfModel* m) { return m->n; }
int nsf_shards(const NsfModel* m) { return m->nsh; }
const NsfTensor* nsf_at(const NsfModel* m, int i) { return i >= 0 && i < m->n ? &m->t[i] : NULL; }
const NsfTensor* nsf_find(const NsfModel* m, const char* name) {
    NsfTensor k;
    if (strlen(name) >= sizeof k.name) return NULL;
    snprintf(k.name, sizeof k.name, "%s", name);
    return m->n ? (const NsfTensor*) bsearch(&k, m->t, (size_t) m->n, sizeof(NsfTensor), tensor_cmp) : NULL;
}
int nsf_mappable(const NsfModel* m, const NsfStream* s) {
    const uint64_t mask = NSF_PAGE - 1;
    return s->off % NSF_PAGE == 0 && s->off + ((s->len + mask) & ~mask) <= (((uint64_t) m->sh[s->shard].size + mask) & ~mask);
}

/* ---------------------------------------------------------------------------------------------------------------------
 * Expert bank files: header (56 bytes, nslm/moe.h:10-17), bias[E] int32, two float[E] error columns, seeds, words and,
 * for P = 4, one exponent code byte a block. */
int nsf_blk_stream(const uint8_t* blk, size_t len, int p, int E, int rows, int cols, int s, uint8_t* dst) {
    enum { HDR = 56 };
    if ((p != 3 && p != 4) || E < 1 || rows < 1 || cols < 8 || s < 0 || s > 3 || (p == 3 && s > 2)) return -1;
    const size_t e = (size_t) E, nb = (size_t) rows * (size_t) cols / 8;
    uint32_t h[3];
    if (len != HDR + 12 * e + (p == 4 ? 5 : 4) * nb * e || memcmp(blk, p == 4 ? "NSLMBLK4" : "NSLMBLKM", 8)) return -1;
    memcpy(h, blk + 8, sizeof h);
    if (h[0] != (uint32_t) rows || h[1] != (uint32_t) cols || h[2] != (uint32_t) E) return -1;
    const uint8_t* base = blk + HDR;
    if (s == 0) memcpy(dst, base + 12 * e, 2 * nb * e);
    else if (s == 1) memcpy(dst, base + 12 * e + 2 * nb * e, 2 * nb * e);
    else if (s == 2) memcpy(dst, base, 4 * e);
    else {
        const uint8_t* ec = base + 12 * e + 4 * nb * e;
        for (size_t k = 0; k < nb * e; k += 2) dst[k / 2] = (uint8_t) ((ec[k] & 15) | ((k + 1 < nb * e ? ec[k + 1] & 15 : 0) << 4));
    }
    return 0;
}

/* ---------------------------------------------------------------------------------------------------------------------
 * Mapping -> HBM through two pinned staging buffers: while one is on its way to the device, the next piece of the
 * mapping is read (page faults and all) into the other. */
#define NSF_STAGE (8u << 20)
int nsf_upload(void* dst_dev, const NsfStream* s, uint64_t skip, uint64_t len) {
    static uint8_t* stage[2];
    static nh_stream_t st;
    static nh_event_t done[2];
    if (skip > s->len || len > s->len - skip) return -1;
    if (!len) return 0;
    if (!stage[0]) {
        if (nh_host_alloc((void**) &stage[0], NSF_STAGE) || nh_host_alloc((void**) &stage[1], NSF_STAGE) || nh_stream_create(&st) ||
            nh_event_create(&done[0]) || nh_event_create(&done[1])) {
            stage[0] = NULL;
            return -1;
        }
    }
    int bad = 0, used[2] = {0, 0};
    uint64_t at = 0;
    for (int i = 0; at < len && !bad; ++i) {
        const int b = i & 1;
        const uint64_t n = len - at < NSF_STAGE ? len - at : NSF_STAGE;
        if (used[b]) bad |= nh_event_sync(done[b]);
        memcpy(stage[b], s->p + skip + at, (size_t) n);
        bad |= nh_memcpy_h2d_async((uint8_t*) dst_dev + at, stage[b], (size_t) n, st);
        bad |= nh_event_record(done[b], st);
        used[b] = 1;
        at += n;
    }
    bad |= nh_stream_sync(st);
    return bad ? -1 : 0;
}
