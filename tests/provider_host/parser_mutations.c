/* Host-side robustness check of the provider's two readers, meant to be built with
 * -fsanitize=address,undefined: every single-byte mutation, truncation and a set of
 * seeded random corruptions of a valid graph document and of a valid SafeTensors file
 * must be either parsed or refused, never read out of bounds.  Arguments: a graph.json
 * and a .safetensors file (small ones), and a scratch path to write mutants to. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "json_min.h"
#include "safetensors_min.h"

static unsigned char* slurp(const char* path, size_t* n) {
    FILE* f = fopen(path, "rb");
    if (!f) return NULL;
    fseek(f, 0, SEEK_END);
    long size = ftell(f);
    fseek(f, 0, SEEK_SET);
    unsigned char* p = (unsigned char*)malloc((size_t)size + 1u);
    if (p && fread(p, 1, (size_t)size, f) != (size_t)size) { free(p); p = NULL; }
    fclose(f);
    if (p) *n = (size_t)size;
    return p;
}

static uint32_t rng_state = 12345u;
static uint32_t rng(void) {
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 17;
    rng_state ^= rng_state << 5;
    return rng_state;
}

static unsigned long json_parsed, json_refused, st_opened, st_refused;

static void try_json(const unsigned char* text, size_t n) {
    const char* error = NULL;
    /* exact-size heap copy, so the sanitizer sees a read one byte past the end */
    char* copy = (char*)malloc(n ? n : 1u);
    memcpy(copy, text, n);
    VxjValue* v = vxj_parse(copy, n, &error);
    if (v) { json_parsed++; vxj_free(v); } else json_refused++;
    free(copy);
}

static void try_safetensors(const unsigned char* bytes, size_t n, const char* scratch) {
    FILE* f = fopen(scratch, "wb");
    if (!f) exit(3);
    fwrite(bytes, 1, n, f);
    fclose(f);
    VxstFile* file = NULL;
    char error[128];
    if (vxst_open(scratch, &file, error, sizeof error) == 0) {
        VxstTensor t;
        static const char* names[] = {"w", "s", "b", "weight", "", "__metadata__"};
        for (size_t i = 0; i < sizeof names / sizeof names[0]; i++) {
            if (vxst_find(file, names[i], &t) && t.bytes) {
                volatile unsigned char first = t.data[0], last = t.data[t.bytes - 1u];
                (void)first; (void)last;
            }
        }
        st_opened++;
        vxst_close(file);
    } else st_refused++;
}

int main(int argc, char** argv) {
    if (argc < 4) return 2;
    size_t jn = 0, sn = 0;
    unsigned char* j = slurp(argv[1], &jn);
    unsigned char* s = slurp(argv[2], &sn);
    if (!j || !s) return 2;
    static const unsigned char pokes[] = {0x00, 0xff, '"', '\\', '{', '}', '[', ']', ',', ':', '-', 'e', '9', 0x80};
    try_json(j, jn);
    for (size_t cut = 0; cut < jn; cut++) try_json(j, cut);
    for (size_t i = 0; i < jn; i++)
        for (size_t p = 0; p < sizeof pokes; p++) {
            unsigned char keep = j[i];
            j[i] = pokes[p];
            try_json(j, jn);
            j[i] = keep;
        }
    /* the SafeTensors header: length word, JSON header, then data */
    uint64_t header = 0;
    memcpy(&header, s, 8);
    const size_t head_end = 8u + (size_t)header < sn ? 8u + (size_t)header : sn;
    try_safetensors(s, sn, argv[3]);
    for (size_t cut = 0; cut <= head_end + 4u && cut < sn; cut += (cut < 16u ? 1u : 7u)) try_safetensors(s, cut, argv[3]);
    for (size_t i = 0; i < head_end; i += (i < 8u ? 1u : 3u))
        for (size_t p = 0; p < sizeof pokes; p += 2) {
            unsigned char keep = s[i];
            s[i] = pokes[p];
            try_safetensors(s, sn, argv[3]);
            s[i] = keep;
        }
    for (int round = 0; round < 400; round++) {
        unsigned char saved[4];
        size_t at[4];
        for (int k = 0; k < 4; k++) {
            at[k] = rng() % head_end;
            saved[k] = s[at[k]];
            s[at[k]] = (unsigned char)rng();
        }
        try_safetensors(s, sn, argv[3]);
        for (int k = 3; k >= 0; k--) s[at[k]] = saved[k];
    }
    printf("json: %lu parsed, %lu refused; safetensors: %lu opened, %lu refused\n", json_parsed, json_refused,
           st_opened, st_refused);
    free(j);
    free(s);
    remove(argv[3]);
    return 0;
}
