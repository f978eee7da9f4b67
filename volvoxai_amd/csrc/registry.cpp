// Kernel-variant table of the hip-gfx950 backend, in the record shape of the
// reference's generated registry (native/src/generated/kernel_registry.h:75-82,
// rows such as "cuda.qlinear.warp-dp4a" at native/src/generated/kernel_registry.c:1171).
// The id chosen for a launch is what the provider reports as route evidence.
#include "../../include/vxhip_w8a8.h"

namespace {
constexpr int kQLinear = 1002, kQGemm = 1005, kQMatMul = 1007, kPackedLinear = 1036;
constexpr int kQuantizeLinear = 0, kDequantizeLinear = 0;  // boundary ops carry no variant rows upstream

#define QROWS(id, entry, pred, feat, prio)            \
    {id, 0, kQLinear, entry, pred, feat, prio},       \
    {id, 0, kQGemm, entry, pred, feat, prio},         \
    {id, 0, kQMatMul, entry, pred, feat, prio}

const VxHipKernelVariant kVariants[] = {
    // (tile suffixes ending in k64 are gemm_k64_kernel, the 16x16x64 form of the large tiles)
    QROWS("hip.qlinear.mfma-i8", "gemm_mfma_kernel<RequantTensor>|gemm_k64_kernel<RequantTensor>",
          "hip.qlinear.canonical-resident-int32-bound-rows-gt32-any-k-tail",
          "hip.gfx950-mfma-i32-32x32x32-i8,hip.gfx950-mfma-i32-16x16x64-i8,hip.global-load-lds-b128", 300),
    QROWS("hip.qlinear.mfma-i8-rowscale", "gemm_mfma_kernel<RequantRow>|gemm_k64_kernel<RequantRow>",
          "hip.qlinear.per-row-input-scale-i8-zero-input-zp-int32-bound-rows-gt32",
          "hip.gfx950-mfma-i32-32x32x32-i8,hip.gfx950-mfma-i32-16x16x64-i8,hip.global-load-lds-b128", 300),
    QROWS("hip.qlinear.gemv-mfma", "gemv_panel_kernel<RequantTensor>",
          "hip.qlinear.canonical-resident-int32-bound-rows-le32",
          "hip.gfx950-mfma-i32-32x32x32-i8,hip.nontemporal-dwordx4", 400),
    QROWS("hip.qlinear.gemv-mfma-rowscale", "gemv_panel_kernel<RequantRow>",
          "hip.qlinear.per-row-input-scale-i8-zero-input-zp-int32-bound-rows-le32",
          "hip.gfx950-mfma-i32-32x32x32-i8,hip.nontemporal-dwordx4", 400),
    {"hip.packed-linear.a8-mfma", 0, kPackedLinear, "gemm_mfma_kernel<DequantF32>|gemm_k64_f32_kernel",
     "hip.packed-linear.w8-dynamic-i8-g32-64-128-256-rows-gt32",
     "hip.gfx950-mfma-i32-32x32x32-i8,hip.gfx950-mfma-i32-16x16x64-i8,hip.global-load-lds-b128", 300},
    {"hip.packed-linear.a8-gemv-mfma", 0, kPackedLinear, "gemv_fit_kernel|gemv_panel_kernel<DequantF32>",
     "hip.packed-linear.w8-dynamic-i8-g32-64-128-256-rows-le32",
     "hip.gfx950-mfma-i32-32x32x32-i8,hip.nontemporal-dwordx4", 400},
    {"hip.packed-linear.w4a8-mfma", 0, kPackedLinear, "gemm_mfma_kernel<DequantF32, W4>|gemm_k64_f32_kernel<W4>",
     "hip.packed-linear.w4-dynamic-i8-g32-64-128-256-rows-gt32",
     "hip.gfx950-mfma-i32-32x32x32-i8,hip.gfx950-mfma-i32-16x16x64-i8,hip.global-load-lds-b128", 300},
    {"hip.packed-linear.w4a8-gemv-mfma", 0, kPackedLinear, "gemv_fit_kernel<W4>|gemv_panel_kernel<DequantF32, W4>",
     "hip.packed-linear.w4-dynamic-i8-g32-64-128-256-rows-le32",
     "hip.gfx950-mfma-i32-32x32x32-i8,hip.nontemporal-dwordx4", 400},
    {"hip.packed-linear.prepare-i8", 0, kPackedLinear, "prepare_i8_kernel|prepare_i8_rows_kernel",
     "hip.packed-linear.dynamic-i8-row-absmax", "", 100},
};
}  // namespace

extern "C" const VxHipKernelVariant* vxhip_kernel_variants(size_t* out_count) {
    (void)kQuantizeLinear;
    (void)kDequantizeLinear;
    if (out_count) *out_count = sizeof(kVariants) / sizeof(kVariants[0]);
    return kVariants;
}
