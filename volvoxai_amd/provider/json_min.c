#include "json_min.h"

#include <errno.h>
#include <stdlib.h>
#include <string.h>

typedef struct Reader {
    const char* p;
    const char* end;
    const char* error;
    int depth;
} Reader;

enum { kMaxDepth = 64 };

static void skip_space(Reader* r) {
    while (r->p < r->end && (*r->p == ' ' || *r->p == '\t' || *r->p == '\n' || *r->p == '\r')) r->p++;
}

static VxjValue* new_value(Reader* r, VxjKind kind) {
    VxjValue* v = (VxjValue*)calloc(1, sizeof(*v));
    if (!v) r->error = "out of memory";
    else v->kind = kind;
    return v;
}

void vxj_free(VxjValue* value) {
    while (value) {
        VxjValue* next = value->next;
        vxj_free(value->first);
        free(value->string);
        free(value->key);
        free(value);
        value = next;
    }
}

static int hex4(const char* p, unsigned* out) {
    unsigned v = 0;
    for (int i = 0; i < 4; i++) {
        char c = p[i];
        v <<= 4;
        if (c >= '0' && c <= '9') v |= (unsigned)(c - '0');
        else if (c >= 'a' && c <= 'f') v |= (unsigned)(c - 'a' + 10);
        else if (c >= 'A' && c <= 'F') v |= (unsigned)(c - 'A' + 10);
        else return 0;
    }
    *out = v;
    return 1;
}

static size_t put_utf8(char* dst, unsigned cp) {
    if (cp < 0x80) { dst[0] = (char)cp; return 1; }
    if (cp < 0x800) { dst[0] = (char)(0xC0 | (cp >> 6)); dst[1] = (char)(0x80 | (cp & 0x3F)); return 2; }
    if (cp < 0x10000) {
        dst[0] = (char)(0xE0 | (cp >> 12));
        dst[1] = (char)(0x80 | ((cp >> 6) & 0x3F));
        dst[2] = (char)(0x80 | (cp & 0x3F));
        return 3;
    }
    dst[0] = (char)(0xF0 | (cp >> 18));
    dst[1] = (char)(0x80 | ((cp >> 12) & 0x3F));
    dst[2] = (char)(0x80 | ((cp >> 6) & 0x3F));
    dst[3] = (char)(0x80 | (cp & 0x3F));
    return 4;
}

/* r->p is at the opening quote. */
static char* parse_string(Reader* r) {
    const char* p = r->p + 1;
    /* the decoded string is never longer than the literal */
    const char* scan = p;
    while (scan < r->end && *scan != '"') {
        if (*scan == '\\') scan++;
        scan++;
    }
    if (scan >= r->end) { r->error = "unterminated string"; return NULL; }
    char* out = (char*)malloc((size_t)(scan - p) + 1u);
    if (!out) { r->error = "out of memory"; return NULL; }
    size_t n = 0;
    while (*p != '"') {
        unsigned char c = (unsigned char)*p;
        if (c < 0x20) { r->error = "control character in string"; free(out); return NULL; }
        if (c != '\\') { out[n++] = (char)c; p++; continue; }
        p++;
        switch (*p) {
            case '"': out[n++] = '"'; p++; break;
            case '\\': out[n++] = '\\'; p++; break;
            case '/': out[n++] = '/'; p++; break;
            case 'b': out[n++] = '\b'; p++; break;
            case 'f': out[n++] = '\f'; p++; break;
            case 'n': out[n++] = '\n'; p++; break;
            case 'r': out[n++] = '\r'; p++; break;
            case 't': out[n++] = '\t'; p++; break;
            case 'u': {
                unsigned cp, low;
                if (r->end - p < 5 || !hex4(p + 1, &cp)) { r->error = "bad \\u escape"; free(out); return NULL; }
                p += 5;
                if (cp >= 0xD800 && cp <= 0xDBFF) {
                    if (r->end - p < 6 || p[0] != '\\' || p[1] != 'u' || !hex4(p + 2, &low) || low < 0xDC00 ||
                        low > 0xDFFF) {
                        r->error = "unpaired surrogate";
                        free(out);
                        return NULL;
                    }
                    cp = 0x10000u + ((cp - 0xD800u) << 10) + (low - 0xDC00u);
                    p += 6;
                } else if (cp >= 0xDC00 && cp <= 0xDFFF) {
                    r->error = "unpaired surrogate";
                    free(out);
                    return NULL;
                }
                if (cp == 0) { r->error = "NUL in string"; free(out); return NULL; }
                n += put_utf8(out + n, cp);
                break;
            }
            default: r->error = "bad escape"; free(out); return NULL;
        }
    }
    out[n] = '\0';
    r->p = p + 1;
    return out;
}

static VxjValue* parse_value(Reader* r);

static VxjValue* parse_number(Reader* r) {
    const char* start = r->p;
    const char* p = start;
    int integral = 1;
    if (p < r->end && *p == '-') p++;
    if (p >= r->end || *p < '0' || *p > '9') { r->error = "bad number"; return NULL; }
    if (*p == '0') p++;
    else while (p < r->end && *p >= '0' && *p <= '9') p++;
    if (p < r->end && *p == '.') {
        integral = 0;
        p++;
        if (p >= r->end || *p < '0' || *p > '9') { r->error = "bad number"; return NULL; }
        while (p < r->end && *p >= '0' && *p <= '9') p++;
    }
    if (p < r->end && (*p == 'e' || *p == 'E')) {
        integral = 0;
        p++;
        if (p < r->end && (*p == '+' || *p == '-')) p++;
        if (p >= r->end || *p < '0' || *p > '9') { r->error = "bad number"; return NULL; }
        while (p < r->end && *p >= '0' && *p <= '9') p++;
    }
    char buffer[64];
    size_t len = (size_t)(p - start);
    if (len >= sizeof(buffer)) { r->error = "number too long"; return NULL; }
    memcpy(buffer, start, len);
    buffer[len] = '\0';
    VxjValue* v = new_value(r, VXJ_NUMBER);
    if (!v) return NULL;
    v->number = strtod(buffer, NULL);
    if (integral) {
        errno = 0;
        long long i = strtoll(buffer, NULL, 10);
        if (errno == 0) {
            v->is_integer = 1;
            v->integer = (int64_t)i;
        }
    }
    r->p = p;
    return v;
}

static int literal(Reader* r, const char* word) {
    size_t n = strlen(word);
    if ((size_t)(r->end - r->p) < n || memcmp(r->p, word, n) != 0) return 0;
    r->p += n;
    return 1;
}

static VxjValue* parse_container(Reader* r, int object) {
    VxjValue* v = new_value(r, object ? VXJ_OBJECT : VXJ_ARRAY);
    VxjValue* tail = NULL;
    const char close = object ? '}' : ']';
    if (!v) return NULL;
    if (++r->depth > kMaxDepth) { r->error = "nesting too deep"; vxj_free(v); return NULL; }
    r->p++;
    skip_space(r);
    if (r->p < r->end && *r->p == close) {
        r->p++;
        r->depth--;
        return v;
    }
    for (;;) {
        char* key = NULL;
        skip_space(r);
        if (object) {
            if (r->p >= r->end || *r->p != '"') { r->error = "object key expected"; break; }
            key = parse_string(r);
            if (!key) break;
            for (const VxjValue* c = v->first; c; c = c->next)
                if (!strcmp(c->key, key)) r->error = "duplicate object key";
            skip_space(r);
            if (r->error || r->p >= r->end || *r->p != ':') {
                if (!r->error) r->error = "':' expected";
                free(key);
                break;
            }
            r->p++;
        }
        VxjValue* child = parse_value(r);
        if (!child) { free(key); break; }
        child->key = key;
        if (tail) tail->next = child; else v->first = child;
        tail = child;
        v->count++;
        skip_space(r);
        if (r->p < r->end && *r->p == ',') { r->p++; continue; }
        if (r->p < r->end && *r->p == close) {
            r->p++;
            r->depth--;
            return v;
        }
        r->error = "',' or closing bracket expected";
        break;
    }
    vxj_free(v);
    return NULL;
}

static VxjValue* parse_value(Reader* r) {
    skip_space(r);
    if (r->p >= r->end) { r->error = "unexpected end"; return NULL; }
    switch (*r->p) {
        case '{': return parse_container(r, 1);
        case '[': return parse_container(r, 0);
        case '"': {
            char* s = parse_string(r);
            if (!s) return NULL;
            VxjValue* v = new_value(r, VXJ_STRING);
            if (!v) { free(s); return NULL; }
            v->string = s;
            return v;
        }
        case 't':
        case 'f': {
            int truth = *r->p == 't';
            if (!literal(r, truth ? "true" : "false")) { r->error = "bad literal"; return NULL; }
            VxjValue* v = new_value(r, VXJ_BOOL);
            if (v) v->boolean = truth;
            return v;
        }
        case 'n':
            if (!literal(r, "null")) { r->error = "bad literal"; return NULL; }
            return new_value(r, VXJ_NULL);
        default: return parse_number(r);
    }
}

VxjValue* vxj_parse(const char* text, size_t length, const char** error) {
    Reader r = {text, text + length, NULL, 0};
    VxjValue* v = parse_value(&r);
    if (v) {
        skip_space(&r);
        if (r.p != r.end) {
            r.error = "trailing text after the document";
            vxj_free(v);
            v = NULL;
        }
    }
    if (error) *error = v ? NULL : (r.error ? r.error : "malformed JSON");
    return v;
}

const VxjValue* vxj_member(const VxjValue* object, const char* key) {
    if (!object || object->kind != VXJ_OBJECT) return NULL;
    for (const VxjValue* c = object->first; c; c = c->next)
        if (!strcmp(c->key, key)) return c;
    return NULL;
}

const VxjValue* vxj_item(const VxjValue* array, size_t index) {
    if (!array || array->kind != VXJ_ARRAY) return NULL;
    const VxjValue* c = array->first;
    while (c && index--) c = c->next;
    return c;
}

const char* vxj_member_string(const VxjValue* object, const char* key) {
    const VxjValue* v = vxj_member(object, key);
    return v && v->kind == VXJ_STRING ? v->string : NULL;
}
