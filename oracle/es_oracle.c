/*
 * CPU oracle for the einsummable apply-node path -- TEST INFRASTRUCTURE ONLY.
 * See es_oracle.h for the list of reference files each part restates.
 *
 * Build:  gcc -O2 -ffp-contract=off -fno-strict-aliasing -fPIC -shared es_oracle.c -lm -o libes_oracle.so
 * (-ffp-contract=off so that float expressions are not fused into FMAs: the reference's
 *  scalar interpreter rounds after every operation.)
 */
#include "es_oracle.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define MAX_RANK 16
#define MAX_INNS 16
#define CHUNK 512

static __thread char g_err[512];

static int fail(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return -1;
}

const char* es_oracle_last_error(void) { return g_err; }

/* ------------------------------------------------------------------ fp16 */

/* IEEE binary16 from double, round-to-nearest-even (half.hpp:373-374 sets
 * HALF_ROUND_STYLE to nearest; ChangeLog: ties to even). */
uint16_t es_oracle_f64_to_f16(double v)
{
    uint64_t b;
    memcpy(&b, &v, 8);
    uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
    int      bexp = (int)((b >> 52) & 0x7ff);
    uint64_t man = b & 0xfffffffffffffULL;
    if (bexp == 0x7ff) {
        return man ? (uint16_t)(sign | 0x7e00u) : (uint16_t)(sign | 0x7c00u);
    }
    if (bexp == 0) {
        return sign; /* zero or a double subnormal, far below 2^-25 */
    }
    int e = bexp - 1023;
    if (e > 15) {
        return (uint16_t)(sign | 0x7c00u);
    }
    man |= (1ULL << 52);
    if (e >= -14) {
        uint64_t m = man >> 42;
        uint64_t rem = man & ((1ULL << 42) - 1);
        uint64_t halfway = 1ULL << 41;
        uint32_t h = (uint32_t)(((uint32_t)(e + 15) << 10) + (uint32_t)(m & 0x3ff));
        if (rem > halfway || (rem == halfway && (h & 1u))) {
            h++;
        }
        return (uint16_t)(sign | h);
    } else {
        int shift = 28 - e; /* value / 2^-24 = man >> shift */
        if (shift > 63) {
            return sign;
        }
        uint64_t m = man >> shift;
        uint64_t rem = man & ((1ULL << shift) - 1);
        uint64_t halfway = 1ULL << (shift - 1);
        if (rem > halfway || (rem == halfway && (m & 1u))) {
            m++;
        }
        return (uint16_t)(sign | (uint16_t)m);
    }
}

uint16_t es_oracle_f32_to_f16(float v) { return es_oracle_f64_to_f16((double)v); }

static double f16_to_f64(uint16_t h)
{
    int      sign = h >> 15;
    int      e = (h >> 10) & 0x1f;
    int      m = h & 0x3ff;
    double   r;
    if (e == 0) {
        r = ldexp((double)m, -24);
    } else if (e == 31) {
        r = m ? NAN : INFINITY;
    } else {
        r = ldexp((double)(m | 0x400), e - 25);
    }
    return sign ? -r : r;
}

float es_oracle_f16_to_f32(uint16_t h) { return (float)f16_to_f64(h); }

static inline double round_f16(double v) { return f16_to_f64(es_oracle_f64_to_f16(v)); }

/* round a double to the value set of a real dtype */
static inline double round_to(int dtype, double v)
{
    switch (dtype) {
        case ES_O_F16:
            return round_f16(v);
        case ES_O_F32:
            return (double)(float)v;
        default:
            return v;
    }
}

static size_t dtype_size(int d) { return d == ES_O_F16 ? 2 : (d == ES_O_F32 ? 4 : 8); }

/* ------------------------------------------------------------- scalarop */

enum {
    K_CONSTANT,
    K_HOLE,
    K_VARIABLE,
    K_ADD,
    K_MUL,
    K_EXP,
    K_LOG,
    K_POWER,
    K_ITE,
    K_CONVERT,
    K_CONJ,
    K_REAL,
    K_IMAG,
    K_CPLEX
};
enum { C_LT, C_GT, C_EQ, C_LE, C_GE };

typedef struct node {
    int          kind;
    int          dtype;
    double       cre, cim; /* constant value (exact in double) */
    int          arg;      /* hole */
    double       power;
    int          compare;
    int          to_dtype;
    char         name[64];
    int          nchild;
    struct node* child[4];
    int          id;
} node_t;

typedef struct {
    node_t* nodes[256];
    int     n;
} tree_t;

static node_t* new_node(tree_t* t)
{
    if (t->n >= 256) {
        fail("scalarop too large");
        return NULL;
    }
    node_t* nd = (node_t*)calloc(1, sizeof(node_t));
    nd->id = t->n;
    t->nodes[t->n++] = nd;
    return nd;
}

static void free_tree(tree_t* t)
{
    for (int i = 0; i != t->n; ++i) {
        free(t->nodes[i]);
    }
    t->n = 0;
}

static int expect(const char** p, const char* s)
{
    size_t n = strlen(s);
    if (strncmp(*p, s, n) != 0) {
        return fail("parse: expected '%s' at '%.20s'", s, *p);
    }
    *p += n;
    return 0;
}

static int parse_dtype(const char** p, int* d)
{
    if (!strncmp(*p, "f16", 3)) {
        *d = ES_O_F16;
    } else if (!strncmp(*p, "f32", 3)) {
        *d = ES_O_F32;
    } else if (!strncmp(*p, "f64", 3)) {
        *d = ES_O_F64;
    } else if (!strncmp(*p, "c64", 3)) {
        *d = ES_O_C64;
    } else {
        return fail("parse: bad dtype at '%.20s'", *p);
    }
    *p += 3;
    return 0;
}

/* scalar_t text: dtype|value with INF / NINF / NAN spelled out (scalarop.cc:2720-2829).
 * Numbers go through the stream extraction of their own type: float for f32, double
 * for f64, double-then-round for f16 (half.hpp:2708-2718), "(re,im)" for c64. */
static int parse_scalar(const char** p, int* dtype, double* re, double* im)
{
    if (parse_dtype(p, dtype)) return -1;
    if (expect(p, "|")) return -1;
    *im = 0.0;
    if (**p == 'I') {
        if (expect(p, "INF")) return -1;
        if (*dtype == ES_O_C64) return fail("parse: complex INF");
        *re = INFINITY;
        return 0;
    }
    if (**p == 'N') {
        if (!strncmp(*p, "NINF", 4)) {
            *p += 4;
            *re = -INFINITY;
        } else if (!strncmp(*p, "NAN", 3)) {
            *p += 3;
            *re = NAN;
        } else {
            return fail("parse: expected NINF or NAN");
        }
        if (*dtype == ES_O_C64) return fail("parse: complex NINF/NAN");
        return 0;
    }
    char* end;
    if (*dtype == ES_O_C64) {
        if (expect(p, "(")) return -1;
        *re = (double)strtof(*p, &end);
        if (end == *p) return fail("parse: bad complex");
        *p = end;
        if (expect(p, ",")) return -1;
        *im = (double)strtof(*p, &end);
        if (end == *p) return fail("parse: bad complex");
        *p = end;
        return expect(p, ")");
    }
    if (*dtype == ES_O_F32) {
        *re = (double)strtof(*p, &end);
    } else if (*dtype == ES_O_F64) {
        *re = strtod(*p, &end);
    } else {
        *re = round_f16(strtod(*p, &end));
    }
    if (end == *p) return fail("parse: bad number at '%.20s'", *p);
    *p = end;
    return 0;
}

static int parse_compare(const char** p, int* c)
{
    char c0 = **p;
    char c1 = (*p)[1];
    if (c0 == '<') {
        *c = (c1 == '=') ? C_LE : C_LT;
        *p += (c1 == '=') ? 2 : 1;
    } else if (c0 == '>') {
        *c = (c1 == '=') ? C_GE : C_GT;
        *p += (c1 == '=') ? 2 : 1;
    } else if (c0 == '=' && c1 == '=') {
        *c = C_EQ;
        *p += 2;
    } else {
        return fail("parse: bad compare");
    }
    return 0;
}

static int num_inputs_of(int kind)
{
    switch (kind) {
        case K_CONSTANT:
        case K_HOLE:
        case K_VARIABLE:
            return 0;
        case K_ADD:
        case K_MUL:
        case K_CPLEX:
            return 2;
        case K_ITE:
            return 4;
        default:
            return 1;
    }
}

/* op_t::type_of (scalarop.cc:775-938); -1 = type failure */
static int type_of(node_t* nd)
{
    int a = nd->nchild > 0 ? nd->child[0]->dtype : -1;
    int b = nd->nchild > 1 ? nd->child[1]->dtype : -1;
    switch (nd->kind) {
        case K_ADD:
        case K_MUL:
            return a == b ? a : -1;
        case K_EXP:
        case K_LOG:
        case K_POWER:
            return a == ES_O_C64 ? -1 : a;
        case K_ITE: {
            int c = nd->child[2]->dtype, d = nd->child[3]->dtype;
            if (a != b || a == ES_O_C64 || c != d) return -1;
            return c;
        }
        case K_CONVERT:
            if (a == ES_O_C64 || nd->to_dtype == ES_O_C64 || a == nd->to_dtype) return -1;
            return nd->to_dtype;
        case K_CONJ:
            return a == ES_O_C64 ? a : -1;
        case K_REAL:
        case K_IMAG:
            return a == ES_O_C64 ? ES_O_F32 : -1;
        case K_CPLEX:
            return (a == b && a == ES_O_F32) ? ES_O_C64 : -1;
    }
    return -1;
}

static node_t* parse_node(tree_t* t, const char** p)
{
    node_t* nd = new_node(t);
    if (!nd) return NULL;
    const char* s = *p;
    if (!strncmp(s, "constant{", 9)) {
        *p += 9;
        nd->kind = K_CONSTANT;
        if (parse_scalar(p, &nd->dtype, &nd->cre, &nd->cim)) return NULL;
        if (expect(p, "}")) return NULL;
    } else if (!strncmp(s, "conj", 4)) {
        *p += 4;
        nd->kind = K_CONJ;
    } else if (!strncmp(s, "complex", 7)) {
        *p += 7;
        nd->kind = K_CPLEX;
    } else if (!strncmp(s, "variable{", 9)) {
        *p += 9;
        nd->kind = K_VARIABLE;
        int i = 0;
        while ((**p >= 'a' && **p <= 'z') || (**p >= 'A' && **p <= 'Z') ||
               (**p >= '0' && **p <= '9') || **p == '_') {
            if (i < 63) nd->name[i++] = **p;
            (*p)++;
        }
        if (expect(p, "|")) return NULL;
        if (parse_dtype(p, &nd->dtype)) return NULL;
        if (expect(p, "}")) return NULL;
    } else if (!strncmp(s, "hole|", 5)) {
        *p += 5;
        nd->kind = K_HOLE;
        if (parse_dtype(p, &nd->dtype)) return NULL;
        if (expect(p, "@")) return NULL;
        char* end;
        nd->arg = (int)strtol(*p, &end, 10);
        if (end == *p) {
            fail("parse: bad hole arg");
            return NULL;
        }
        *p = end;
    } else if (*s == '+') {
        *p += 1;
        nd->kind = K_ADD;
    } else if (*s == '*') {
        *p += 1;
        nd->kind = K_MUL;
    } else if (!strncmp(s, "exp", 3)) {
        *p += 3;
        nd->kind = K_EXP;
    } else if (!strncmp(s, "log", 3)) {
        *p += 3;
        nd->kind = K_LOG;
    } else if (!strncmp(s, "power{", 6)) {
        *p += 6;
        nd->kind = K_POWER;
        char* end;
        nd->power = strtod(*p, &end);
        if (end == *p) {
            fail("parse: bad power");
            return NULL;
        }
        *p = end;
        if (expect(p, "}")) return NULL;
    } else if (!strncmp(s, "ite_", 4)) {
        *p += 4;
        nd->kind = K_ITE;
        if (parse_compare(p, &nd->compare)) return NULL;
    } else if (!strncmp(s, "imag", 4)) {
        *p += 4;
        nd->kind = K_IMAG;
    } else if (!strncmp(s, "to_", 3)) {
        *p += 3;
        nd->kind = K_CONVERT;
        if (parse_dtype(p, &nd->to_dtype)) return NULL;
    } else if (!strncmp(s, "real", 4)) {
        *p += 4;
        nd->kind = K_REAL;
    } else {
        fail("parse: unknown op at '%.20s'", s);
        return NULL;
    }

    int n = num_inputs_of(nd->kind);
    if (n == 0) return nd;
    if (expect(p, "[")) return NULL;
    for (int i = 0; i != n; ++i) {
        if (i > 0 && expect(p, ",")) return NULL;
        nd->child[i] = parse_node(t, p);
        if (!nd->child[i]) return NULL;
        nd->nchild++;
    }
    if (expect(p, "]")) return NULL;
    nd->dtype = type_of(nd);
    if (nd->dtype < 0) {
        fail("type failure in node parse");
        return NULL;
    }
    return nd;
}

static node_t* parse_scalarop(tree_t* t, const char* text)
{
    const char* p = text;
    t->n = 0;
    node_t* root = parse_node(t, &p);
    if (!root) {
        free_tree(t);
        return NULL;
    }
    if (*p != 0) {
        fail("parse: trailing text '%.20s'", p);
        free_tree(t);
        return NULL;
    }
    return root;
}

static const char* dtype_str(int d)
{
    static const char* s[] = {"f16", "f32", "f64", "c64"};
    return s[d];
}
static const char* compare_str(int c)
{
    static const char* s[] = {"<", ">", "==", "<=", ">="};
    return s[c];
}

typedef struct {
    char*  buf;
    size_t cap, len;
    int    overflow;
} sbuf_t;

static void sb_printf(sbuf_t* sb, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    size_t room = sb->cap > sb->len ? sb->cap - sb->len : 0;
    int    n = vsnprintf(sb->buf + (room ? sb->len : 0), room, fmt, ap);
    va_end(ap);
    if (n < 0 || (size_t)n >= room) {
        sb->overflow = 1;
    } else {
        sb->len += (size_t)n;
    }
}

/* default ostream formatting of a floating value == printf("%g") (precision 6) */
static void sb_number(sbuf_t* sb, double v)
{
    if (isinf(v)) {
        sb_printf(sb, v > 0 ? "INF" : "NINF");
    } else if (isnan(v)) {
        sb_printf(sb, "NAN");
    } else {
        sb_printf(sb, "%g", v);
    }
}

static void print_node(sbuf_t* sb, node_t const* nd)
{
    switch (nd->kind) {
        case K_CONSTANT:
            sb_printf(sb, "constant{%s|", dtype_str(nd->dtype));
            if (nd->dtype == ES_O_C64) {
                sb_printf(sb, "(%g,%g)", nd->cre, nd->cim);
            } else {
                sb_number(sb, nd->cre);
            }
            sb_printf(sb, "}");
            break;
        case K_HOLE:
            sb_printf(sb, "hole|%s@%d", dtype_str(nd->dtype), nd->arg);
            break;
        case K_VARIABLE:
            sb_printf(sb, "variable{%s|%s}", nd->name, dtype_str(nd->dtype));
            break;
        case K_ADD:
            sb_printf(sb, "+");
            break;
        case K_MUL:
            sb_printf(sb, "*");
            break;
        case K_EXP:
            sb_printf(sb, "exp");
            break;
        case K_LOG:
            sb_printf(sb, "log");
            break;
        case K_POWER:
            sb_printf(sb, "power{%g}", nd->power);
            break;
        case K_ITE:
            sb_printf(sb, "ite_%s", compare_str(nd->compare));
            break;
        case K_CONVERT:
            sb_printf(sb, "to_%s", dtype_str(nd->to_dtype));
            break;
        case K_CONJ:
            sb_printf(sb, "conj");
            break;
        case K_REAL:
            sb_printf(sb, "real");
            break;
        case K_IMAG:
            sb_printf(sb, "imag");
            break;
        case K_CPLEX:
            sb_printf(sb, "complex");
            break;
    }
    if (nd->nchild) {
        sb_printf(sb, "[");
        for (int i = 0; i != nd->nchild; ++i) {
            if (i) sb_printf(sb, ",");
            print_node(sb, nd->child[i]);
        }
        sb_printf(sb, "]");
    }
}

int es_oracle_scalarop_roundtrip(const char* text, char* out, size_t cap)
{
    tree_t  t;
    node_t* root = parse_scalarop(&t, text);
    if (!root) return -1;
    sbuf_t sb = {out, cap, 0, 0};
    print_node(&sb, root);
    free_tree(&t);
    if (sb.overflow) return fail("roundtrip: buffer too small");
    return 0;
}

static int collect_holes(node_t const* nd, int* dt, int cap)
{
    if (nd->kind == K_HOLE) {
        if (nd->arg < 0 || nd->arg >= cap) return fail("hole arg out of range");
        if (dt[nd->arg] >= 0 && dt[nd->arg] != nd->dtype) {
            return fail("hole %d used with two dtypes", nd->arg);
        }
        dt[nd->arg] = nd->dtype;
    }
    for (int i = 0; i != nd->nchild; ++i) {
        if (collect_holes(nd->child[i], dt, cap)) return -1;
    }
    return 0;
}

static int has_variable(node_t const* nd)
{
    if (nd->kind == K_VARIABLE) return 1;
    for (int i = 0; i != nd->nchild; ++i) {
        if (has_variable(nd->child[i])) return 1;
    }
    return 0;
}

int es_oracle_scalarop_info(const char* text, int* out_dtype, int* n_inputs, int* inn_dtypes,
                            int cap)
{
    tree_t  t;
    node_t* root = parse_scalarop(&t, text);
    if (!root) return -1;
    int dt[MAX_INNS];
    for (int i = 0; i != MAX_INNS; ++i) dt[i] = -1;
    int rc = collect_holes(root, dt, MAX_INNS);
    *out_dtype = root->dtype;
    int n = 0;
    for (int i = 0; i != MAX_INNS; ++i) {
        if (dt[i] >= 0) n = i + 1;
    }
    *n_inputs = n;
    for (int i = 0; i != n && i < cap; ++i) inn_dtypes[i] = dt[i];
    free_tree(&t);
    return rc;
}

/* Chunked evaluation.  Every node produces n values; a value is held as a double (and a
 * second double for the imaginary part of c64), which represents f16/f32 values exactly.
 *
 * EXACT mode follows op_t::_eval_* (scalarop.cc:641-780): the operation is performed in the
 * node's own dtype.  f16 results are the correctly rounded binary16 value of the exact
 * result (half 2.2.0 arithmetic is correctly rounded for + and *; for exp/log/pow the double
 * result rounded once is used).  f32 uses float arithmetic and expf/logf/powf with the
 * exponent cast to float (scalarop.cc:719-720); f16 pow rounds the exponent to f16 first
 * (scalarop.cc:716-717).
 *
 * WIDE mode evaluates every node in double with no intermediate rounding. */
typedef struct {
    double* re; /* [n_nodes][CHUNK] */
    double* im;
    double const* const* inn_re;
    double const* const* inn_im;
    int mode;
} evalctx_t;

static int do_compare(int c, double a, double b)
{
    switch (c) {
        case C_LT:
            return a < b;
        case C_GT:
            return a > b;
        case C_EQ:
            return a == b;
        case C_LE:
            return a <= b;
        default:
            return a >= b;
    }
}

static int eval_node(evalctx_t* cx, node_t const* nd, int n)
{
    double* re = cx->re + (size_t)nd->id * CHUNK;
    double* im = cx->im + (size_t)nd->id * CHUNK;
    for (int i = 0; i != nd->nchild; ++i) {
        if (eval_node(cx, nd->child[i], n)) return -1;
    }
    double const* are = nd->nchild > 0 ? cx->re + (size_t)nd->child[0]->id * CHUNK : NULL;
    double const* aim = nd->nchild > 0 ? cx->im + (size_t)nd->child[0]->id * CHUNK : NULL;
    double const* bre = nd->nchild > 1 ? cx->re + (size_t)nd->child[1]->id * CHUNK : NULL;
    double const* bim = nd->nchild > 1 ? cx->im + (size_t)nd->child[1]->id * CHUNK : NULL;
    int const exact = cx->mode == ES_O_EXACT;
    int const dt = nd->dtype;
    switch (nd->kind) {
        case K_CONSTANT:
            for (int i = 0; i != n; ++i) {
                re[i] = nd->cre;
                im[i] = nd->cim;
            }
            return 0;
        case K_HOLE:
            memcpy(re, cx->inn_re[nd->arg], sizeof(double) * (size_t)n);
            if (dt == ES_O_C64) memcpy(im, cx->inn_im[nd->arg], sizeof(double) * (size_t)n);
            return 0;
        case K_VARIABLE:
            return fail("cannot evaluate a scalarop with variables");
        case K_ADD:
            if (dt == ES_O_C64) {
                for (int i = 0; i != n; ++i) {
                    if (exact) {
                        re[i] = (double)((float)are[i] + (float)bre[i]);
                        im[i] = (double)((float)aim[i] + (float)bim[i]);
                    } else {
                        re[i] = are[i] + bre[i];
                        im[i] = aim[i] + bim[i];
                    }
                }
            } else if (!exact || dt == ES_O_F64) {
                for (int i = 0; i != n; ++i) re[i] = are[i] + bre[i];
            } else if (dt == ES_O_F32) {
                for (int i = 0; i != n; ++i) re[i] = (double)((float)are[i] + (float)bre[i]);
            } else {
                for (int i = 0; i != n; ++i) re[i] = round_f16(are[i] + bre[i]);
            }
            return 0;
        case K_MUL:
            if (dt == ES_O_C64) {
                for (int i = 0; i != n; ++i) {
                    if (exact) {
                        float a = (float)are[i], b = (float)aim[i];
                        float c = (float)bre[i], d = (float)bim[i];
                        float ac = a * c, bd = b * d, ad = a * d, bc = b * c;
                        re[i] = (double)(ac - bd);
                        im[i] = (double)(ad + bc);
                    } else {
                        re[i] = are[i] * bre[i] - aim[i] * bim[i];
                        im[i] = are[i] * bim[i] + aim[i] * bre[i];
                    }
                }
            } else if (!exact || dt == ES_O_F64) {
                for (int i = 0; i != n; ++i) re[i] = are[i] * bre[i];
            } else if (dt == ES_O_F32) {
                for (int i = 0; i != n; ++i) re[i] = (double)((float)are[i] * (float)bre[i]);
            } else {
                for (int i = 0; i != n; ++i) re[i] = round_f16(are[i] * bre[i]);
            }
            return 0;
        case K_EXP:
            if (!exact || dt == ES_O_F64) {
                for (int i = 0; i != n; ++i) re[i] = exp(are[i]);
            } else if (dt == ES_O_F32) {
                for (int i = 0; i != n; ++i) re[i] = (double)expf((float)are[i]);
            } else {
                for (int i = 0; i != n; ++i) re[i] = round_f16(exp(are[i]));
            }
            return 0;
        case K_LOG:
            if (!exact || dt == ES_O_F64) {
                for (int i = 0; i != n; ++i) re[i] = log(are[i]);
            } else if (dt == ES_O_F32) {
                for (int i = 0; i != n; ++i) re[i] = (double)logf((float)are[i]);
            } else {
                for (int i = 0; i != n; ++i) re[i] = round_f16(log(are[i]));
            }
            return 0;
        case K_POWER: {
            double p = nd->power;
            if (dt == ES_O_F16) p = round_f16(p);
            if (dt == ES_O_F32) p = (double)(float)p;
            if (!exact || dt == ES_O_F64) {
                for (int i = 0; i != n; ++i) re[i] = pow(are[i], p);
            } else if (dt == ES_O_F32) {
                for (int i = 0; i != n; ++i) re[i] = (double)powf((float)are[i], (float)p);
            } else {
                for (int i = 0; i != n; ++i) re[i] = round_f16(pow(are[i], p));
            }
            return 0;
        }
        case K_ITE: {
            double const* tre = cx->re + (size_t)nd->child[2]->id * CHUNK;
            double const* tim = cx->im + (size_t)nd->child[2]->id * CHUNK;
            double const* fre = cx->re + (size_t)nd->child[3]->id * CHUNK;
            double const* fim = cx->im + (size_t)nd->child[3]->id * CHUNK;
            for (int i = 0; i != n; ++i) {
                int c = do_compare(nd->compare, are[i], bre[i]);
                re[i] = c ? tre[i] : fre[i];
                if (dt == ES_O_C64) im[i] = c ? tim[i] : fim[i];
            }
            return 0;
        }
        case K_CONVERT:
            if (exact) {
                for (int i = 0; i != n; ++i) re[i] = round_to(dt, are[i]);
            } else {
                for (int i = 0; i != n; ++i) re[i] = are[i];
            }
            return 0;
        case K_CONJ:
            for (int i = 0; i != n; ++i) {
                re[i] = are[i];
                im[i] = -aim[i];
            }
            return 0;
        case K_REAL:
            for (int i = 0; i != n; ++i) re[i] = are[i];
            return 0;
        case K_IMAG:
            for (int i = 0; i != n; ++i) re[i] = aim[i];
            return 0;
        case K_CPLEX:
            for (int i = 0; i != n; ++i) {
                re[i] = are[i];
                im[i] = bre[i];
            }
            return 0;
    }
    return fail("eval: bad node");
}

/* typed load/store of element i of a dense array */
static inline void load_elem(int dtype, const void* p, uint64_t i, double* re, double* im)
{
    switch (dtype) {
        case ES_O_F16:
            *re = f16_to_f64(((const uint16_t*)p)[i]);
            break;
        case ES_O_F32:
            *re = (double)((const float*)p)[i];
            break;
        case ES_O_F64:
            *re = ((const double*)p)[i];
            break;
        default:
            *re = (double)((const float*)p)[2 * i];
            *im = (double)((const float*)p)[2 * i + 1];
    }
}
static inline void store_elem(int dtype, void* p, uint64_t i, double re, double im)
{
    switch (dtype) {
        case ES_O_F16:
            ((uint16_t*)p)[i] = es_oracle_f64_to_f16(re);
            break;
        case ES_O_F32:
            ((float*)p)[i] = (float)re;
            break;
        case ES_O_F64:
            ((double*)p)[i] = re;
            break;
        default:
            ((float*)p)[2 * i] = (float)re;
            ((float*)p)[2 * i + 1] = (float)im;
    }
}

typedef struct {
    tree_t   tree;
    node_t*  root;
    int      n_inputs;
    int      inn_dtypes[MAX_INNS];
    double*  node_re;
    double*  node_im;
    double*  in_re[MAX_INNS];
    double*  in_im[MAX_INNS];
} program_t;

static void program_free(program_t* pg)
{
    free(pg->node_re);
    free(pg->node_im);
    for (int i = 0; i != MAX_INNS; ++i) {
        free(pg->in_re[i]);
        free(pg->in_im[i]);
    }
    free_tree(&pg->tree);
}

static int program_init(program_t* pg, const char* text)
{
    memset(pg, 0, sizeof(*pg));
    pg->root = parse_scalarop(&pg->tree, text);
    if (!pg->root) return -1;
    for (int i = 0; i != MAX_INNS; ++i) pg->inn_dtypes[i] = -1;
    if (collect_holes(pg->root, pg->inn_dtypes, MAX_INNS)) {
        free_tree(&pg->tree);
        return -1;
    }
    if (has_variable(pg->root)) {
        free_tree(&pg->tree);
        return fail("cannot evaluate a scalarop with variables");
    }
    pg->n_inputs = 0;
    for (int i = 0; i != MAX_INNS; ++i) {
        if (pg->inn_dtypes[i] >= 0) pg->n_inputs = i + 1;
    }
    pg->node_re = (double*)malloc(sizeof(double) * CHUNK * (size_t)pg->tree.n);
    pg->node_im = (double*)calloc(CHUNK * (size_t)pg->tree.n, sizeof(double));
    for (int i = 0; i != pg->n_inputs; ++i) {
        pg->in_re[i] = (double*)malloc(sizeof(double) * CHUNK);
        pg->in_im[i] = (double*)calloc(CHUNK, sizeof(double));
    }
    return 0;
}

/* evaluate n <= CHUNK points whose inputs sit in pg->in_re/in_im; results in *re,*im */
static int program_run(program_t* pg, int n, int mode, double const** re, double const** im)
{
    evalctx_t cx;
    cx.re = pg->node_re;
    cx.im = pg->node_im;
    cx.inn_re = (double const* const*)pg->in_re;
    cx.inn_im = (double const* const*)pg->in_im;
    cx.mode = mode;
    if (eval_node(&cx, pg->root, n)) return -1;
    *re = pg->node_re + (size_t)pg->root->id * CHUNK;
    *im = pg->node_im + (size_t)pg->root->id * CHUNK;
    return 0;
}

static void bits_to_value(int dtype, uint64_t bits, double* re, double* im)
{
    unsigned char raw[8];
    memcpy(raw, &bits, 8);
    *im = 0;
    switch (dtype) {
        case ES_O_F16: {
            uint16_t h;
            memcpy(&h, raw, 2);
            *re = f16_to_f64(h);
            break;
        }
        case ES_O_F32: {
            float f;
            memcpy(&f, raw, 4);
            *re = (double)f;
            break;
        }
        case ES_O_F64:
            memcpy(re, raw, 8);
            break;
        default: {
            float c[2];
            memcpy(c, raw, 8);
            *re = (double)c[0];
            *im = (double)c[1];
        }
    }
}

static uint64_t value_to_bits(int dtype, double re, double im)
{
    uint64_t bits = 0;
    switch (dtype) {
        case ES_O_F16: {
            uint16_t h = es_oracle_f64_to_f16(re);
            memcpy(&bits, &h, 2);
            break;
        }
        case ES_O_F32: {
            float f = (float)re;
            memcpy(&bits, &f, 4);
            break;
        }
        case ES_O_F64:
            memcpy(&bits, &re, 8);
            break;
        default: {
            float c[2] = {(float)re, (float)im};
            memcpy(&bits, c, 8);
        }
    }
    return bits;
}

int es_oracle_scalarop_eval(const char* text, int n_inputs, const uint64_t* input_bits, int mode,
                            uint64_t* out_bits, int* out_dtype)
{
    program_t pg;
    if (program_init(&pg, text)) return -1;
    if (n_inputs < pg.n_inputs) {
        program_free(&pg);
        return fail("eval: %d inputs given, %d needed", n_inputs, pg.n_inputs);
    }
    for (int k = 0; k != pg.n_inputs; ++k) {
        if (pg.inn_dtypes[k] < 0) continue;
        bits_to_value(pg.inn_dtypes[k], input_bits[k], &pg.in_re[k][0], &pg.in_im[k][0]);
    }
    double const *re, *im;
    int rc = program_run(&pg, 1, mode, &re, &im);
    if (!rc) {
        *out_bits = value_to_bits(pg.root->dtype, re[0], im[0]);
        *out_dtype = pg.root->dtype;
    }
    program_free(&pg);
    return rc;
}

int es_oracle_scalarop_map(const char* text, int n_inputs, const void* const* inputs, uint64_t n,
                           int mode, void* out)
{
    program_t pg;
    if (program_init(&pg, text)) return -1;
    if (n_inputs < pg.n_inputs) {
        program_free(&pg);
        return fail("map: %d inputs given, %d needed", n_inputs, pg.n_inputs);
    }
    int rc = 0;
    for (uint64_t b = 0; b < n && !rc; b += CHUNK) {
        int m = (int)((n - b) < CHUNK ? (n - b) : CHUNK);
        for (int k = 0; k != pg.n_inputs; ++k) {
            if (pg.inn_dtypes[k] < 0) continue;
            for (int i = 0; i != m; ++i) {
                load_elem(pg.inn_dtypes[k], inputs[k], b + (uint64_t)i, &pg.in_re[k][i],
                          &pg.in_im[k][i]);
            }
        }
        double const *re, *im;
        rc = program_run(&pg, m, mode, &re, &im);
        if (rc) break;
        for (int i = 0; i != m; ++i) store_elem(pg.root->dtype, out, b + (uint64_t)i, re[i], im[i]);
    }
    program_free(&pg);
    return rc;
}

/* ---------------------------------------------------------- einsummable */

typedef struct {
    int      join_rank, out_rank, n_inns;
    uint64_t join_shape[MAX_RANK];
    int      inn_rank[MAX_INNS];
    int      inn[MAX_INNS][MAX_RANK];
} es_t;

/* constructor checks + aggregation renumbering (einsummable.cc:32-93, 538-584) */
static int es_init(es_t* e, const uint64_t* join_shape, int join_rank, const int* inns_flat,
                   const int* inns_offsets, int n_inns, int out_rank)
{
    if (join_rank < 1 || join_rank > MAX_RANK) return fail("einsummable: bad join rank");
    if (n_inns < 1 || n_inns > MAX_INNS) return fail("einsummable: bad number of inputs");
    if (out_rank < 1) return fail("einsummable: invalid inns, out rank");
    e->join_rank = join_rank;
    e->out_rank = out_rank;
    e->n_inns = n_inns;
    for (int k = 0; k != n_inns; ++k) {
        int r = inns_offsets[k + 1] - inns_offsets[k];
        if (r < 1 || r > MAX_RANK) return fail("compute_join_rank: empty inn given");
        e->inn_rank[k] = r;
        for (int i = 0; i != r; ++i) e->inn[k][i] = inns_flat[inns_offsets[k] + i];
    }
    /* renumber aggregation modes in order of first appearance */
    {
        int agg_cnt = out_rank;
        int fix[4 * MAX_RANK];
        for (int i = 0; i != 4 * MAX_RANK; ++i) fix[i] = -1;
        for (int k = 0; k != n_inns; ++k) {
            for (int i = 0; i != e->inn_rank[k]; ++i) {
                int m = e->inn[k][i];
                if (m < 0 || m >= 4 * MAX_RANK) return fail("einsummable: bad mode id");
                if (m >= out_rank) {
                    if (fix[m] < 0) fix[m] = agg_cnt++;
                    e->inn[k][i] = fix[m];
                }
            }
        }
    }
    int almost = 0;
    for (int k = 0; k != n_inns; ++k) {
        for (int i = 0; i != e->inn_rank[k]; ++i) {
            if (e->inn[k][i] > almost) almost = e->inn[k][i];
        }
    }
    almost += 1;
    int jr = almost > out_rank ? almost : out_rank;
    if (jr != join_rank) return fail("invalid join shape size");
    for (int i = 0; i != join_rank; ++i) {
        if (join_shape[i] == 0) return fail("einsummable: cannot have zero join size");
        e->join_shape[i] = join_shape[i];
    }
    for (int k = 0; k != n_inns; ++k) {
        for (int i = 0; i != e->inn_rank[k]; ++i) {
            for (int j = i + 1; j != e->inn_rank[k]; ++j) {
                if (e->inn[k][i] == e->inn[k][j]) {
                    return fail("einsummable: invalid inns, out rank");
                }
            }
        }
    }
    return 0;
}

static char castable_check(char c)
{
    return (c == '+' || c == 'x' || c == 'v' || c == '^') ? c : 0;
}

int es_oracle_einsummable(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                          const int* inns_offsets, int n_inns, int out_rank, const char* join_text,
                          char castable, int mode, void* out, const void* const* inns)
{
    es_t e;
    if (es_init(&e, join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank)) return -1;
    int has_agg = out_rank < join_rank;
    if (has_agg && !castable_check(castable)) {
        return fail("Must have castable when aggregating.");
    }
    program_t pg;
    if (program_init(&pg, join_text)) return -1;
    if (pg.n_inputs != n_inns) {
        program_free(&pg);
        return fail("einsummable inns size not same as scalarop join");
    }
    for (int k = 0; k != n_inns; ++k) {
        if (pg.inn_dtypes[k] < 0) {
            program_free(&pg);
            return fail("einsummable does not use all of its inputs!");
        }
    }
    int const odt = pg.root->dtype;
    if ((castable == 'v' || castable == '^') && odt == ES_O_C64 && has_agg) {
        program_free(&pg);
        return fail("cannot min/max complex");
    }

    /* stride of every join mode inside every (row-major) input */
    uint64_t stride[MAX_INNS][MAX_RANK];
    for (int k = 0; k != n_inns; ++k) {
        for (int m = 0; m != join_rank; ++m) stride[k][m] = 0;
        uint64_t s = 1;
        for (int i = e.inn_rank[k] - 1; i >= 0; --i) {
            stride[k][e.inn[k][i]] = s;
            s *= e.join_shape[e.inn[k][i]];
        }
    }
    uint64_t n_out = 1, n_agg = 1;
    for (int i = 0; i != out_rank; ++i) n_out *= e.join_shape[i];
    for (int i = out_rank; i != join_rank; ++i) n_agg *= e.join_shape[i];

    uint64_t* base = (uint64_t*)malloc(sizeof(uint64_t) * CHUNK * (size_t)n_inns);
    double*   acc_re = (double*)malloc(sizeof(double) * CHUNK);
    double*   acc_im = (double*)calloc(CHUNK, sizeof(double));
    int       rc = 0;

    for (uint64_t o0 = 0; o0 < n_out && !rc; o0 += CHUNK) {
        int n = (int)((n_out - o0) < CHUNK ? (n_out - o0) : CHUNK);
        /* per out element: offset of the (agg = 0) element in every input */
        for (int i = 0; i != n; ++i) {
            uint64_t rem = o0 + (uint64_t)i;
            uint64_t off[MAX_INNS] = {0};
            for (int m = out_rank - 1; m >= 0; --m) {
                uint64_t d = rem % e.join_shape[m];
                rem /= e.join_shape[m];
                for (int k = 0; k != n_inns; ++k) off[k] += d * stride[k][m];
            }
            for (int k = 0; k != n_inns; ++k) base[(size_t)k * CHUNK + i] = off[k];
        }
        uint64_t agg_idx[MAX_RANK] = {0};
        for (uint64_t a = 0; a != n_agg; ++a) {
            for (int k = 0; k != n_inns; ++k) {
                uint64_t aoff = 0;
                for (int m = out_rank; m != join_rank; ++m) aoff += agg_idx[m] * stride[k][m];
                for (int i = 0; i != n; ++i) {
                    load_elem(pg.inn_dtypes[k], inns[k], base[(size_t)k * CHUNK + i] + aoff,
                              &pg.in_re[k][i], &pg.in_im[k][i]);
                }
            }
            double const *re, *im;
            rc = program_run(&pg, n, mode, &re, &im);
            if (rc) break;
            if (a == 0) {
                /* initialisation with the first aggregation index (reference.cc:456-462) */
                memcpy(acc_re, re, sizeof(double) * (size_t)n);
                if (odt == ES_O_C64) memcpy(acc_im, im, sizeof(double) * (size_t)n);
            } else {
                /* agg_into: castable scalarop evaluated in the output dtype
                 * (dbuffer.cc:343-347; make_min/make_max scalarop.cc:2267-2280) */
                int exact = mode == ES_O_EXACT;
                for (int i = 0; i != n; ++i) {
                    double x = acc_re[i], y = re[i];
                    switch (castable) {
                        case '+':
                            if (odt == ES_O_C64) {
                                if (exact) {
                                    acc_re[i] = (double)((float)x + (float)y);
                                    acc_im[i] = (double)((float)acc_im[i] + (float)im[i]);
                                } else {
                                    acc_re[i] = x + y;
                                    acc_im[i] += im[i];
                                }
                            } else {
                                if (exact && odt == ES_O_F32) {
                                    acc_re[i] = (double)((float)x + (float)y);
                                } else {
                                    acc_re[i] = exact ? round_to(odt, x + y) : x + y;
                                }
                            }
                            break;
                        case 'x':
                            if (odt == ES_O_C64) {
                                double xi = acc_im[i], yi = im[i];
                                if (exact) {
                                    float ac = (float)x * (float)y, bd = (float)xi * (float)yi;
                                    float ad = (float)x * (float)yi, bc = (float)xi * (float)y;
                                    acc_re[i] = (double)(ac - bd);
                                    acc_im[i] = (double)(ad + bc);
                                } else {
                                    acc_re[i] = x * y - xi * yi;
                                    acc_im[i] = x * yi + xi * y;
                                }
                            } else if (exact && odt == ES_O_F32) {
                                acc_re[i] = (double)((float)x * (float)y);
                            } else {
                                acc_re[i] = exact ? round_to(odt, x * y) : x * y;
                            }
                            break;
                        case 'v':
                            acc_re[i] = (x < y) ? x : y;
                            break;
                        case '^':
                            acc_re[i] = (x > y) ? x : y;
                            break;
                    }
                }
            }
            /* row-major increment over the aggregated modes */
            for (int m = join_rank - 1; m >= out_rank; --m) {
                if (++agg_idx[m] < e.join_shape[m]) break;
                agg_idx[m] = 0;
            }
        }
        if (rc) break;
        for (int i = 0; i != n; ++i) store_elem(odt, out, o0 + (uint64_t)i, acc_re[i], acc_im[i]);
    }
    free(base);
    free(acc_re);
    free(acc_im);
    program_free(&pg);
    return rc;
}

/* update_count_adjacent / build_adjacents (einsummable.cc:95-164): for mode r find how many
 * consecutive modes r, r+1, ... can be fused: in every term they must either all be absent or
 * appear adjacent and in order. */
static int count_adjacent(const int* is, int n, int pos)
{
    int cnt = 0;
    int v = is[pos];
    while (pos != n && is[pos] == v) {
        ++pos;
        ++v;
        ++cnt;
    }
    return cnt;
}
static int find_mode(const int* is, int n, int r)
{
    for (int i = 0; i != n; ++i) {
        if (is[i] == r) return i;
    }
    return -1;
}

int es_oracle_merge_adjacent_dims(const uint64_t* join_shape, int join_rank, const int* inns_flat,
                                  const int* inns_offsets, int n_inns, int out_rank,
                                  uint64_t* new_join_shape, int* new_inns_flat,
                                  int* new_inns_offsets, int* new_out_rank)
{
    es_t e;
    if (es_init(&e, join_shape, join_rank, inns_flat, inns_offsets, n_inns, out_rank)) return -1;
    /* terms = inputs followed by the output (0..out_rank-1) */
    int nt = n_inns + 1;
    int term[MAX_INNS + 1][MAX_RANK];
    int term_rank[MAX_INNS + 1];
    for (int k = 0; k != n_inns; ++k) {
        term_rank[k] = e.inn_rank[k];
        memcpy(term[k], e.inn[k], sizeof(int) * MAX_RANK);
    }
    term_rank[n_inns] = out_rank;
    for (int i = 0; i != out_rank; ++i) term[n_inns][i] = i;

    int group_begin[MAX_RANK], group_end[MAX_RANK], n_groups = 0;
    int r = 0;
    while (r != join_rank) {
        int score = 0;
        int first = -1;
        for (int k = 0; k != nt && score == 0; ++k) {
            int pos = find_mode(term[k], term_rank[k], r);
            if (pos >= 0) {
                score = count_adjacent(term[k], term_rank[k], pos);
                first = k;
            }
        }
        if (score <= 0) return fail("merge_adjacent_dims: mode %d unused", r);
        for (int k = 0; k != nt; ++k) {
            if (k == first) continue;
            int pos = find_mode(term[k], term_rank[k], r);
            if (pos < 0) {
                int end = r + score;
                for (int i = 0; i != term_rank[k]; ++i) {
                    int m = term[k][i];
                    if (m >= r && m < end) end = m;
                }
                score = end - r;
            } else {
                int c = count_adjacent(term[k], term_rank[k], pos);
                if (c < score) score = c;
            }
        }
        if (score <= 0) return fail("impl err");
        group_begin[n_groups] = r;
        group_end[n_groups] = r + score;
        ++n_groups;
        r += score;
    }
    int backwards[MAX_RANK];
    for (int w = 0; w != n_groups; ++w) {
        uint64_t sz = 1;
        for (int i = group_begin[w]; i != group_end[w]; ++i) {
            sz *= e.join_shape[i];
            backwards[i] = w;
        }
        new_join_shape[w] = sz;
    }
    int pos = 0;
    for (int k = 0; k != nt; ++k) {
        if (k < n_inns) new_inns_offsets[k] = pos;
        int i = 0, cnt = 0;
        while (i != term_rank[k]) {
            int w = backwards[term[k][i]];
            if (k < n_inns) new_inns_flat[pos++] = w;
            ++cnt;
            i += group_end[w] - group_begin[w];
        }
        if (k == n_inns) *new_out_rank = cnt;
    }
    new_inns_offsets[n_inns] = pos;
    return n_groups;
}

int es_oracle_einsummable_str(const int* inns_flat, const int* inns_offsets, int n_inns,
                              int out_rank, char* out, size_t cap)
{
    sbuf_t sb = {out, cap, 0, 0};
    /* same renumbering as the constructor */
    int agg_cnt = out_rank;
    int fix[4 * MAX_RANK];
    for (int i = 0; i != 4 * MAX_RANK; ++i) fix[i] = -1;
    for (int k = 0; k != n_inns; ++k) {
        if (k) sb_printf(&sb, ",");
        for (int i = inns_offsets[k]; i != inns_offsets[k + 1]; ++i) {
            int m = inns_flat[i];
            if (m < 0 || m >= 4 * MAX_RANK) return fail("bad mode id");
            if (m >= out_rank) {
                if (fix[m] < 0) fix[m] = agg_cnt++;
                m = fix[m];
            }
            sb_printf(&sb, "%c", 'a' + m);
        }
    }
    sb_printf(&sb, "->");
    for (int i = 0; i != out_rank; ++i) sb_printf(&sb, "%c", 'a' + i);
    return sb.overflow ? fail("str: buffer too small") : 0;
}

int es_oracle_einsummable_parse(const char* str, int* inns_flat, int* inns_offsets, int* n_inns,
                                int* out_rank, int cap)
{
    const char* arrow = strstr(str, "->");
    if (!arrow) return fail("invalid einsummable parse: no arrow");
    const char* outw = arrow + 2;
    int         orank = (int)strlen(outw);
    if (orank == 0) return fail("invalid parse: empty out");
    int map[256];
    for (int i = 0; i != 256; ++i) map[i] = -1;
    int cnt = 0;
    for (int i = 0; i != orank; ++i) {
        unsigned char c = (unsigned char)outw[i];
        if (c == '-' || c == ',') return fail("invalid parse: bad character in output");
        if (map[c] >= 0) return fail("output in einsummable cannot have duplicates");
        map[c] = cnt++;
    }
    int k = 0, pos = 0;
    inns_offsets[0] = 0;
    for (const char* p = str; p != arrow; ++p) {
        unsigned char c = (unsigned char)*p;
        if (c == ',') {
            if (pos == inns_offsets[k]) return fail("invalid einsummable parse: empty after comma");
            inns_offsets[++k] = pos;
        } else {
            if (map[c] < 0) map[c] = cnt++;
            if (pos >= cap) return fail("parse: too many modes");
            inns_flat[pos++] = map[c];
        }
    }
    if (pos == inns_offsets[k]) return fail("invalid einsummable parse: empty inn after arrow");
    inns_offsets[++k] = pos;
    *n_inns = k;
    *out_rank = orank;
    return 0;
}

/* ---------------------------------------------------------------- touch */

int es_oracle_touch_simplify(const uint64_t* dims, int rank, uint64_t* out_dims, int* out_rank)
{
    if (rank < 1) return fail("touch: empty selection");
    int n = 1;
    memcpy(out_dims, dims, sizeof(uint64_t) * 5);
    for (int i = 1; i != rank; ++i) {
        const uint64_t* td = dims + 5 * i;
        int dummy = td[0] == td[1] && td[2] == 0 && td[3] == 0 && td[0] == td[4];
        if (dummy) {
            uint64_t  d = td[0];
            uint64_t* b = out_dims + 5 * (n - 1);
            for (int j = 0; j != 5; ++j) b[j] *= d;
        } else {
            memcpy(out_dims + 5 * n, td, sizeof(uint64_t) * 5);
            ++n;
        }
    }
    *out_rank = n;
    return 0;
}

/* _reference_touch (reference.cc:565-590) with the update functions of
 * reference.cc:522-562 / engine/touch.cc:119-135 (std::min / std::max semantics:
 * min keeps `out` unless inn < out; max keeps `out` unless out < inn). */
int es_oracle_touch(const uint64_t* dims, int rank, char castable, int dtype, void* out,
                    const void* inn)
{
    if (rank < 1 || rank > MAX_RANK) return fail("touch: bad rank");
    if (castable && !castable_check(castable)) return fail("touch: bad castable");
    if (dtype == ES_O_C64 && (castable == 'v' || castable == '^')) {
        return fail("ref touch update complex not implemented");
    }
    uint64_t total = 1;
    for (int i = 0; i != rank; ++i) {
        const uint64_t* td = dims + 5 * i;
        if (td[2] + td[4] > td[0] || td[3] + td[4] > td[1]) return fail("touch: out of range");
        total *= td[4];
    }
    uint64_t idx[MAX_RANK] = {0};
    size_t   esz = dtype_size(dtype);
    for (uint64_t t = 0; t != total; ++t) {
        uint64_t ii = 0, io = 0;
        for (int i = 0; i != rank; ++i) {
            const uint64_t* td = dims + 5 * i;
            ii = ii * td[0] + (idx[i] + td[2]);
            io = io * td[1] + (idx[i] + td[3]);
        }
        if (!castable) {
            memcpy((char*)out + io * esz, (const char*)inn + ii * esz, esz);
        } else {
            double vr = 0, vi = 0, ar = 0, ai = 0;
            load_elem(dtype, out, io, &vr, &vi);
            load_elem(dtype, inn, ii, &ar, &ai);
            double rr = vr, ri = vi;
            switch (castable) {
                case '+':
                    if (dtype == ES_O_F32 || dtype == ES_O_C64) {
                        rr = (double)((float)vr + (float)ar);
                        ri = (double)((float)vi + (float)ai);
                    } else {
                        rr = vr + ar; /* f16: exact in double, rounded once by store_elem */
                    }
                    break;
                case 'x':
                    if (dtype == ES_O_C64) {
                        float ac = (float)vr * (float)ar, bd = (float)vi * (float)ai;
                        float ad = (float)vr * (float)ai, bc = (float)vi * (float)ar;
                        rr = (double)(ac - bd);
                        ri = (double)(ad + bc);
                    } else if (dtype == ES_O_F32) {
                        rr = (double)((float)vr * (float)ar);
                    } else {
                        rr = vr * ar;
                    }
                    break;
                case 'v':
                    rr = (ar < vr) ? ar : vr;
                    break;
                case '^':
                    rr = (vr < ar) ? ar : vr;
                    break;
            }
            if ((castable == 'v' || castable == '^')) {
                /* min/max select one of the operands: copy its bits */
                int take_inn = (castable == 'v') ? (ar < vr) : (vr < ar);
                if (take_inn) memcpy((char*)out + io * esz, (const char*)inn + ii * esz, esz);
            } else {
                store_elem(dtype, out, io, rr, ri);
            }
        }
        for (int i = rank - 1; i >= 0; --i) {
            if (++idx[i] < dims[5 * i + 4]) break;
            idx[i] = 0;
        }
    }
    return 0;
}

/* ---------------------------------------------------------------- fills */

int es_oracle_fill_constant(int dtype, uint64_t bits, uint64_t nelem, void* out)
{
    size_t esz = dtype_size(dtype);
    for (uint64_t i = 0; i != nelem; ++i) memcpy((char*)out + i * esz, &bits, esz);
    return 0;
}

/* reference_fill (reference.cc:491-503): ret[i,j] = (i - start >= j) ? lower : upper with
 * signed i - start. */
int es_oracle_fill_lowertri(int dtype, uint64_t lower_bits, uint64_t upper_bits, uint64_t nrow,
                            uint64_t ncol, int64_t start, void* out)
{
    size_t esz = dtype_size(dtype);
    for (int64_t i = 0; i != (int64_t)nrow; ++i) {
        for (int64_t j = 0; j != (int64_t)ncol; ++j) {
            uint64_t const* src = (i - start >= j) ? &lower_bits : &upper_bits;
            memcpy((char*)out + ((uint64_t)i * ncol + (uint64_t)j) * esz, src, esz);
        }
    }
    return 0;
}
