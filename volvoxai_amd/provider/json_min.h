/* A small strict JSON reader for graph.json and SafeTensors headers: whole
 * document into a tree, UTF-8 strings with the standard escapes, numbers as
 * double plus an exact int64 when the literal is an integer.  Duplicate object
 * keys and trailing text are errors, as a strict package loader wants them. */
#ifndef VXHIP_PROVIDER_JSON_MIN_H
#define VXHIP_PROVIDER_JSON_MIN_H

#include <stddef.h>
#include <stdint.h>

typedef enum VxjKind {
    VXJ_NULL = 0,
    VXJ_BOOL,
    VXJ_NUMBER,
    VXJ_STRING,
    VXJ_ARRAY,
    VXJ_OBJECT
} VxjKind;

typedef struct VxjValue {
    VxjKind kind;
    int boolean;
    double number;
    int is_integer;       /* the literal had no fraction/exponent and fits int64 */
    int64_t integer;
    char* string;         /* VXJ_STRING: NUL-terminated (embedded NULs are rejected) */
    char* key;            /* set when this value is an object member */
    struct VxjValue* first;  /* children of an array/object, in document order */
    struct VxjValue* next;
    size_t count;
} VxjValue;

/* Returns NULL and a static message in *error on malformed input. */
VxjValue* vxj_parse(const char* text, size_t length, const char** error);
void vxj_free(VxjValue* value);

const VxjValue* vxj_member(const VxjValue* object, const char* key);
const VxjValue* vxj_item(const VxjValue* array, size_t index);
/* String content of a VXJ_STRING member, else NULL. */
const char* vxj_member_string(const VxjValue* object, const char* key);

#endif
