/* Read-only view of SafeTensors files: an 8-byte little-endian header length,
 * a JSON header {"name": {"dtype", "shape", "data_offsets": [begin, end]}, ...,
 * "__metadata__": {...}}, then the tensor bytes.  The file is memory-mapped;
 * tensor pointers stay valid until vxst_close. */
#ifndef VXHIP_PROVIDER_SAFETENSORS_MIN_H
#define VXHIP_PROVIDER_SAFETENSORS_MIN_H

#include <stddef.h>
#include <stdint.h>

#define VXST_MAX_RANK 8u

typedef struct VxstTensor {
    char dtype[8];            /* "I8", "U8", "I32", "U32", "F32", ... */
    uint32_t rank;
    int64_t shape[VXST_MAX_RANK];
    const uint8_t* data;
    size_t bytes;
} VxstTensor;

typedef struct VxstFile VxstFile;

/* 0 on success; otherwise a message is written to error. */
int vxst_open(const char* path, VxstFile** out, char* error, size_t error_capacity);
void vxst_close(VxstFile* file);
/* 1 and *out filled if the file holds a tensor of that name, else 0. */
int vxst_find(const VxstFile* file, const char* name, VxstTensor* out);
/* 1 when the file's __metadata__ object has the key. */
int vxst_metadata_has(const VxstFile* file, const char* key);

#endif
