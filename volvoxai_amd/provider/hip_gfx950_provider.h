/* Source-level composition, as for any provider of the reference runtime
 * (docs/backend-sdk.md:60-73): link this object with the host program and
 * libvxhip_w8a8, call the register function once before CreateRuntime. */
#ifndef VOLVOXAI_HIP_GFX950_PROVIDER_H
#define VOLVOXAI_HIP_GFX950_PROVIDER_H

#include "volvoxai_backend.h"

#ifdef __cplusplus
extern "C" {
#endif

VX_API VxStatus volvoxai_hip_gfx950_backend_register(VxReport* report);

/* What compile would make of a package, decided without touching a device. */
VX_API VxStatus volvoxai_hip_gfx950_inspect_package(const VxModelSource* source,
                                                    VxPackedArithmetic arithmetic,
                                                    uint32_t* d_in, uint32_t* d_out,
                                                    int32_t* is_packed_linear,
                                                    char* message, size_t message_capacity);

#ifdef __cplusplus
}
#endif

#endif
