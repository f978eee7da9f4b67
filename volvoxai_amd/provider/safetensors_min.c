#include "safetensors_min.h"

#include "json_min.h"

#include <fcntl.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

struct VxstFile {
    uint8_t* map;
    size_t map_bytes;
    const uint8_t* payload;
    size_t payload_bytes;
    VxjValue* header;
};

static size_t dtype_bytes(const char* dtype) {
    static const struct { const char* name; size_t bytes; } table[] = {
        {"BOOL", 1}, {"U8", 1}, {"I8", 1}, {"F8_E5M2", 1}, {"F8_E4M3", 1}, {"I16", 2}, {"U16", 2},
        {"F16", 2}, {"BF16", 2}, {"I32", 4}, {"U32", 4}, {"F32", 4}, {"F64", 8}, {"I64", 8}, {"U64", 8},
    };
    for (size_t i = 0; i < sizeof(table) / sizeof(table[0]); i++)
        if (!strcmp(table[i].name, dtype)) return table[i].bytes;
    return 0;
}

static int fail(char* error, size_t cap, const char* what, const char* path) {
    if (error && cap) snprintf(error, cap, "%s: %s", what, path ? path : "");
    return -1;
}

int vxst_open(const char* path, VxstFile** out, char* error, size_t cap) {
    struct stat st;
    uint64_t header_bytes = 0;
    const char* json_error = NULL;
    if (!path || !out) return fail(error, cap, "null argument", path);
    *out = NULL;
    int fd = open(path, O_RDONLY);
    if (fd < 0) return fail(error, cap, "cannot open weight file", path);
    if (fstat(fd, &st) != 0 || st.st_size < 8) {
        close(fd);
        return fail(error, cap, "weight file is shorter than a SafeTensors header", path);
    }
    VxstFile* f = (VxstFile*)calloc(1, sizeof(*f));
    if (!f) {
        close(fd);
        return fail(error, cap, "out of memory", path);
    }
    f->map_bytes = (size_t)st.st_size;
    f->map = (uint8_t*)mmap(NULL, f->map_bytes, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (f->map == MAP_FAILED) {
        free(f);
        return fail(error, cap, "cannot map weight file", path);
    }
    for (int i = 7; i >= 0; i--) header_bytes = (header_bytes << 8) | f->map[i];
    if (header_bytes > f->map_bytes - 8u) {
        vxst_close(f);
        return fail(error, cap, "SafeTensors header length exceeds the file", path);
    }
    f->header = vxj_parse((const char*)f->map + 8, (size_t)header_bytes, &json_error);
    if (!f->header || f->header->kind != VXJ_OBJECT) {
        vxst_close(f);
        return fail(error, cap, json_error ? json_error : "SafeTensors header is not an object", path);
    }
    f->payload = f->map + 8 + header_bytes;
    f->payload_bytes = f->map_bytes - 8u - (size_t)header_bytes;
    *out = f;
    return 0;
}

void vxst_close(VxstFile* f) {
    if (!f) return;
    if (f->map && f->map != MAP_FAILED) munmap(f->map, f->map_bytes);
    vxj_free(f->header);
    free(f);
}

int vxst_find(const VxstFile* f, const char* name, VxstTensor* out) {
    if (!f || !name || !out || !strcmp(name, "__metadata__")) return 0;
    const VxjValue* entry = vxj_member(f->header, name);
    if (!entry || entry->kind != VXJ_OBJECT) return 0;
    const char* dtype = vxj_member_string(entry, "dtype");
    const VxjValue* shape = vxj_member(entry, "shape");
    const VxjValue* offsets = vxj_member(entry, "data_offsets");
    if (!dtype || strlen(dtype) >= sizeof(out->dtype) || !shape || shape->kind != VXJ_ARRAY ||
        shape->count > VXST_MAX_RANK || !offsets || offsets->kind != VXJ_ARRAY || offsets->count != 2)
        return 0;
    const VxjValue* b = vxj_item(offsets, 0);
    const VxjValue* e = vxj_item(offsets, 1);
    if (b->kind != VXJ_NUMBER || e->kind != VXJ_NUMBER || !b->is_integer || !e->is_integer ||
        b->integer < 0 || e->integer < b->integer || (uint64_t)e->integer > f->payload_bytes)
        return 0;
    memset(out, 0, sizeof(*out));
    snprintf(out->dtype, sizeof(out->dtype), "%s", dtype);
    out->rank = (uint32_t)shape->count;
    uint64_t elements = 1;
    size_t axis = 0;
    for (const VxjValue* d = shape->first; d; d = d->next, axis++) {
        if (d->kind != VXJ_NUMBER || !d->is_integer || d->integer < 0) return 0;
        out->shape[axis] = d->integer;
        if (d->integer && elements > UINT64_MAX / (uint64_t)d->integer) return 0;
        elements *= (uint64_t)d->integer;
    }
    const size_t element_bytes = dtype_bytes(dtype);
    out->bytes = (size_t)(e->integer - b->integer);
    if (!element_bytes || elements > UINT64_MAX / element_bytes || elements * element_bytes != out->bytes) return 0;
    out->data = f->payload + b->integer;
    return 1;
}

int vxst_metadata_has(const VxstFile* f, const char* key) {
    if (!f || !key) return 0;
    const VxjValue* metadata = vxj_member(f->header, "__metadata__");
    return metadata && metadata->kind == VXJ_OBJECT && vxj_member(metadata, key) != NULL;
}
