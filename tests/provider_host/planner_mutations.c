/* Host-side robustness check of the provider's package reading beyond the two file readers: the
 * graph planner (tensor table, ports, node order, fused linears, the decoder route), meant to be
 * built with -fsanitize=address,undefined together with the provider's own sources.  A valid
 * package is read once (it must be accepted), then its graph document is mutated -- truncations,
 * single-byte pokes at every position, digit and name edits, seeded random corruptions -- and every
 * mutant must be either accepted or refused with a status; the sanitizers abort on the first read
 * or write out of bounds, use after free or undefined operation.  No device is touched: the
 * provider's inspect entry reads a package exactly as compile does and stops before the upload.
 *
 * Arguments: arithmetic (the VxPackedArithmetic value), a scratch path for mutants, the graph.json,
 * then one or more SafeTensors files. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "volvoxai_backend.h"

VxStatus volvoxai_hip_gfx950_inspect_package(const VxModelSource* source, VxPackedArithmetic arithmetic, uint32_t* d_in,
                                             uint32_t* d_out, int32_t* is_packed_linear, char* message,
                                             size_t message_capacity);

/* the provider registers itself with the host it is linked into; this program is that host */
VxStatus vx_backend_register_provider(const VxBackendProvider* provider, VxReport* report) {
    (void)provider;
    (void)report;
    return VX_STATUS_OK;
}

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

static uint32_t rng_state = 2463534242u;
static uint32_t rng(void) {
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 17;
    rng_state ^= rng_state << 5;
    return rng_state;
}

static unsigned long accepted, refused;
static const char* scratch;
static const char** weights;
static size_t weight_count;
static VxPackedArithmetic arithmetic;

static VxStatus inspect_bytes(const unsigned char* text, size_t n) {
    FILE* f = fopen(scratch, "wb");
    if (!f) exit(3);
    fwrite(text, 1, n, f);
    fclose(f);
    VxModelSource source;
    memset(&source, 0, sizeof source);
    source.struct_size = sizeof source;
    source.graph_path = scratch;
    source.weight_paths = weights;
    source.weight_path_count = weight_count;
    uint32_t d_in = 0, d_out = 0;
    int32_t packed = 0;
    char message[256];
    message[0] = 0;
    const VxStatus st = volvoxai_hip_gfx950_inspect_package(&source, arithmetic, &d_in, &d_out, &packed, message,
                                                            sizeof message);
    if (st == VX_STATUS_OK) accepted++; else refused++;
    return st;
}

int main(int argc, char** argv) {
    if (argc < 5) return 2;
    arithmetic = (VxPackedArithmetic)atoi(argv[1]);
    scratch = argv[2];
    weights = (const char**)&argv[4];
    weight_count = (size_t)(argc - 4);
    size_t n = 0;
    unsigned char* g = slurp(argv[3], &n);
    if (!g) return 2;
    if (inspect_bytes(g, n) != VX_STATUS_OK) {
        fprintf(stderr, "the unmutated package was refused\n");
        return 4;
    }
    /* truncations: sparse through the body, dense near the end */
    for (size_t cut = 0; cut < n; cut += (n - cut > 64u ? 17u : 1u)) inspect_bytes(g, cut);
    /* single-byte pokes: structure characters, digits, a sign, a letter, a high byte */
    static const unsigned char pokes[] = {'"', '{', '}', '[', ']', ',', ':', '-', '0', '9', 'e', 'x', 0x00, 0x80};
    const size_t stride = n > 2400u ? n / 1200u : 1u;  /* about 1200 positions of a large document */
    for (size_t i = 0; i < n; i += stride)
        for (size_t p = 0; p < sizeof pokes; p++) {
            if (g[i] == pokes[p]) continue;
            const unsigned char keep = g[i];
            g[i] = pokes[p];
            inspect_bytes(g, n);
            g[i] = keep;
        }
    /* every digit run changed: to zero, to a huge number, to a negative one (shapes, group sizes, counts) */
    for (size_t i = 0; i < n; i++) {
        if (g[i] < '0' || g[i] > '9' || (i && g[i - 1] >= '0' && g[i - 1] <= '9')) continue;
        size_t end = i;
        while (end < n && g[end] >= '0' && g[end] <= '9') end++;
        static const char* subs[] = {"0", "4294967297", "-3", "1e9", "7"};
        for (size_t s = 0; s < sizeof subs / sizeof subs[0]; s++) {
            const size_t sl = strlen(subs[s]);
            unsigned char* m = (unsigned char*)malloc(n - (end - i) + sl + 1u);
            memcpy(m, g, i);
            memcpy(m + i, subs[s], sl);
            memcpy(m + i + sl, g + end, n - end);
            inspect_bytes(m, n - (end - i) + sl);
            free(m);
        }
    }
    /* names: one character of every string changed, so that references stop resolving or start to collide */
    for (size_t i = 1; i + 1 < n; i++) {
        if (g[i - 1] != '"' || g[i] == '"') continue;
        const unsigned char keep = g[i];
        g[i] = keep == 'q' ? 'r' : 'q';
        inspect_bytes(g, n);
        g[i] = keep;
    }
    /* seeded random corruptions, four bytes at a time */
    for (int round = 0; round < 1500; round++) {
        unsigned char saved[4];
        size_t at[4];
        for (int k = 0; k < 4; k++) {
            at[k] = rng() % n;
            saved[k] = g[at[k]];
            g[at[k]] = (unsigned char)rng();
        }
        inspect_bytes(g, n);
        for (int k = 3; k >= 0; k--) g[at[k]] = saved[k];
    }
    printf("packages: %lu accepted, %lu refused\n", accepted, refused);
    free(g);
    remove(scratch);
    return 0;
}
