/* Backend provider "hip-gfx950": plugs libvxhip_w8a8 into the unchanged
 * VolvoxAI runtime through its provider SPI (native/include/volvoxai_backend.h:168-259).
 *
 * The provider compiles W8A8 packages whose graph is one node or a chain of nodes, each reading
 * the tensor the one before it wrote (one graph input, one graph output):
 *   - QLinear / QGemm / QMatMul in the volvox-affine-safetensors/v1
 *     representation (docs/w8a8-safetensors.md:13-59, validation list :158-175);
 *   - PackedLinear with weight_bits 8, 4, 3 or 2 under DYNAMIC_I8 packed
 *     arithmetic (node form: native/tests/test_packed_arithmetic.inc:35-37);
 *   - QuantizeLinear / DequantizeLinear with per-tensor parameters (node form: inputs
 *     input, scale, zero_point; python/tests/test_transpose_quantization_dynamic.py:29-37).
 * Intermediate tensors of a chain stay in device memory.  Anything else is refused with BACKEND_UNSUPPORTED before a compiled instance
 * exists, which is what shape_domain.support = FULL promises
 * (native/include/volvoxai_backend.h:112-118).
 *
 * Ownership follows docs/backend-sdk.md:77-95: the runtime instance names the
 * device, the compiled instance holds the immutable prepacked weights, every
 * context instance owns its stream, staging buffers and scratch, so contexts of
 * one compiled model may execute concurrently
 * (native/tests/test_packed_arithmetic.inc:128-147).
 */
#include "hip_gfx950_provider.h"

#include "json_min.h"
#include "safetensors_min.h"
#include "vxhip_w8a8.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define PROVIDER_NAME "hip-gfx950"
#define NAME_CAPACITY 256u

typedef struct HipRuntime {
    int32_t device;
    char device_name[VX_REPORT_DEVICE_CAPACITY];
} HipRuntime;

typedef enum PlanKind {
    PLAN_QLINEAR = 1,
    PLAN_PACKED_LINEAR = 2,
    PLAN_QUANTIZE = 3,
    PLAN_DEQUANTIZE = 4,
    PLAN_REQUANTIZE = 5
} PlanKind;

#define MAX_CHAIN_NODES 64u
#define MAX_GRAPH_PORTS 8u                           /* graph inputs, and graph outputs */
#define MAX_GRAPH_TENSORS (MAX_CHAIN_NODES + MAX_GRAPH_PORTS) /* every graph input and node output */

/* Host-side result of reading one node; tensor pointers borrow the mapped weight files, which
 * belong to the ChainPlan. */
typedef struct PackagePlan {
    PlanKind kind;
    char node_id[NAME_CAPACITY];
    char input_name[NAME_CAPACITY];
    char output_name[NAME_CAPACITY];
    uint32_t d_in, d_out;
    VxDataType input_dtype, output_dtype;
    uint32_t input_slot, output_slot; /* the tensors it reads and writes, as indices of the graph's tensor table */
    /* QLinear */
    const void* weight;
    uint32_t weight_dtype;
    const float* weight_scales;
    int32_t* weight_zero_points; /* owned */
    const int32_t* bias_i32;
    float input_scale, output_scale;
    int32_t input_zero_point, output_zero_point;
    /* PackedLinear */
    const uint32_t* packed_words;
    const float* group_scales;
    const float* bias_f32;
    uint32_t group_size;
    uint32_t weight_bits;
    /* QuantizeLinear / DequantizeLinear: parameters of the byte side */
    float boundary_scale;
    int32_t boundary_zero_point;
    /* Aligned copies of the small F32/I32 payloads above (scales, biases): a SafeTensors payload
     * starts wherever its header ends and may be misaligned for its element type. */
    void* aligned_copies[4];
    size_t aligned_count;
    /* mapped files (borrowed) */
    VxstFile** files;
    size_t file_count;
} PackagePlan;

/* A tensor of the graph: a graph input or the output of a node.  All share their leading extents
 * (the rows); name, element type and last extent tell them apart. */
typedef struct PlanTensor {
    char name[NAME_CAPACITY];
    VxDataType dtype;
    uint32_t d;
} PlanTensor;

/* The whole graph: its nodes in execution order (every node reads a graph input or the output of
 * an earlier node -- a chain, a tree with shared prefixes, several independent branches), the
 * tensors between them and the files they read.  input_name .. output_dtype describe the first
 * graph input and the first graph output. */
typedef struct ChainPlan {
    PackagePlan* nodes;
    size_t count;
    VxstFile** files;
    size_t file_count;
    PlanTensor tensors[MAX_GRAPH_TENSORS];
    size_t tensor_count;
    uint32_t input_slots[MAX_GRAPH_PORTS], output_slots[MAX_GRAPH_PORTS];
    size_t input_count, output_count;
    char input_name[NAME_CAPACITY];
    char output_name[NAME_CAPACITY];
    uint32_t d_in, d_out;
    VxDataType input_dtype, output_dtype;
    int any_packed;
} ChainPlan;

/* One compiled node. */
typedef struct HipStage {
    PlanKind kind;
    uint32_t input_slot, output_slot;
    uint32_t d_in, d_out;
    VxDataType input_dtype, output_dtype;
    VxHipQLinear* qlinear;
    VxHipPackedLinear* packed;
    float input_scale, output_scale; /* QLinear; the byte side of a boundary node in input_scale */
    int32_t input_zero_point, output_zero_point;
    /* A QLinear whose bytes only a DequantizeLinear reads runs both in one launch and writes that
     * node's f32 tensor (dequantized_slot); the DequantizeLinear stage is then marked absorbed. */
    int dequantizes, absorbed;
    /* ... and one whose input bytes only it reads, written by a QuantizeLinear with the linear's own input
     * parameters, starts from that node's f32 tensor (quantized_slot; the QuantizeLinear is absorbed) */
    int quantizes;
    uint32_t quantized_slot;
    const char* family; /* of the launch, for the route string */
    uint32_t dequantized_slot;
    float dequantize_scale;
    int32_t dequantize_zero_point;
} HipStage;

struct DecoderModel;
struct DecoderState;

typedef struct HipCompiled {
    HipRuntime* runtime;
    struct DecoderModel* decoder; /* set for a decoder graph (decoder_route.inc); stages are then unused */
    HipStage* stages;
    size_t stage_count;
    PlanTensor tensors[MAX_GRAPH_TENSORS]; /* graph inputs and node outputs; a context holds one device buffer each */
    size_t tensor_count;
    uint32_t input_slots[MAX_GRAPH_PORTS], output_slots[MAX_GRAPH_PORTS];
    size_t input_count, output_count;
    uint64_t widest_row_bytes;  /* of any tensor of the graph */
    uint64_t all_rows_bytes;    /* of one row of every tensor together */
    uint64_t widest_float_row;  /* elements of the widest PackedLinear input (its int8 staging) */
    uint32_t rank;                        /* of every input and output alike */
    int64_t lead_min[VX_MAX_TENSOR_RANK]; /* bounds of the leading dimensions */
    int64_t lead_max[VX_MAX_TENSOR_RANK];
    int64_t lead_multiple[VX_MAX_TENSOR_RANK];
    /* Scheduler batching: possible when axis 0 is a symbolic axis that admits extent 1 and the
     * core proved the requests independent along it; the identities are echoed in the contract. */
    int batch_capable;
    char graph_fingerprint[256];
    char batch_proof_identity[256];
    char route[128];
} HipCompiled;

typedef struct HipContext {
    HipCompiled* compiled;
    VxHipContext* ctx;
    struct DecoderState* decode; /* decoder graphs: the cache and work buffers of this context */
    void* tensor_dev[MAX_GRAPH_TENSORS]; /* one buffer per tensor of the graph, grown to the rows of a call */
    size_t tensor_capacity[MAX_GRAPH_TENSORS];
    void* output_host[MAX_GRAPH_PORTS];
    size_t host_capacity[MAX_GRAPH_PORTS];
    int closed;
} HipContext;

/* ---- reports ---------------------------------------------------------------- */

static int report_writable(const VxReport* report) {
    return report && report->struct_size == sizeof(*report);
}

static void fill_report(VxReport* report, const HipRuntime* runtime, VxStatus status, VxStage stage,
                        VxOperationCode code, const char* message) {
    if (!report_writable(report)) return;
    memset(report, 0, sizeof(*report));
    report->struct_size = sizeof(*report);
    report->status = status;
    report->stage = stage;
    report->code = code;
    snprintf(report->backend, sizeof(report->backend), "%s", PROVIDER_NAME);
    snprintf(report->device, sizeof(report->device), "%s",
             runtime && runtime->device_name[0] ? runtime->device_name : "gfx950");
    snprintf(report->message, sizeof(report->message), "%s", message ? message : "");
}

static VxOperationCode code_for(VxStatus status) {
    switch (status) {
        case VX_STATUS_OK: return VX_CODE_NONE;
        case VX_STATUS_OUT_OF_MEMORY: return VX_CODE_OUT_OF_MEMORY;
        case VX_STATUS_BACKEND_UNSUPPORTED: return VX_CODE_BACKEND_UNSUPPORTED;
        case VX_STATUS_BACKEND_UNAVAILABLE: return VX_CODE_BACKEND_UNAVAILABLE;
        case VX_STATUS_DEVICE_LOST: return VX_CODE_DEVICE_LOST;
        case VX_STATUS_INVALID_GRAPH: return VX_CODE_INVALID_GRAPH;
        case VX_STATUS_EXECUTION_FAILED: return VX_CODE_DEVICE_EXECUTION_FAILED;
        default: return VX_CODE_INVALID_ARGUMENT;
    }
}

static void attest(VxReport* report, size_t nodes, const char* route) {
    if (!report_writable(report)) return;
    report->route_attested = 1;
    report->operator_fallback_used = 0;
    snprintf(report->route_evidence, sizeof(report->route_evidence), "provider=%s;nodes=%zu;route=%s", PROVIDER_NAME,
             nodes, route);
    snprintf(report->fallback_evidence, sizeof(report->fallback_evidence), "%s", "operator=none");
}

/* ---- package reading ------------------------------------------------------------ */

typedef struct Failure {
    VxStatus status;
    char message[VX_REPORT_MESSAGE_CAPACITY];
} Failure;

static VxStatus refuse(Failure* failure, VxStatus status, const char* format, const char* detail) {
    failure->status = status;
    snprintf(failure->message, sizeof(failure->message), format, detail ? detail : "");
    return status;
}

static void chain_release(ChainPlan* chain) {
    for (size_t i = 0; i < chain->count; i++) {
        free(chain->nodes[i].weight_zero_points);
        for (size_t c = 0; c < chain->nodes[i].aligned_count; c++) free(chain->nodes[i].aligned_copies[c]);
    }
    free(chain->nodes);
    for (size_t i = 0; i < chain->file_count; i++) vxst_close(chain->files[i]);
    free(chain->files);
    memset(chain, 0, sizeof(*chain));
}

static char* read_text_file(const char* path, size_t* length) {
    FILE* file = path ? fopen(path, "rb") : NULL;
    long size;
    char* bytes;
    if (!file) return NULL;
    if (fseek(file, 0, SEEK_END) != 0 || (size = ftell(file)) < 0 || fseek(file, 0, SEEK_SET) != 0) {
        fclose(file);
        return NULL;
    }
    bytes = (char*)malloc((size_t)size + 1u);
    if (bytes && fread(bytes, 1, (size_t)size, file) != (size_t)size) {
        free(bytes);
        bytes = NULL;
    }
    fclose(file);
    if (bytes) {
        bytes[size] = '\0';
        *length = (size_t)size;
    }
    return bytes;
}

/* A tensor name must resolve in exactly one of the bound weight files
 * (docs/w8a8-safetensors.md:103-108). */
static int find_tensor(const PackagePlan* plan, const char* name, VxstTensor* out) {
    int found = 0;
    for (size_t i = 0; i < plan->file_count; i++) {
        VxstTensor t;
        if (vxst_find(plan->files[i], name, &t)) {
            if (found) return -1;
            *out = t;
            found = 1;
        }
    }
    return found;
}

static int copy_name(char* dst, const char* src) {
    if (!src || !src[0] || strlen(src) >= NAME_CAPACITY) return 0;
    memcpy(dst, src, strlen(src) + 1u);
    return 1;
}

static int graph_dtype(const char* text, VxDataType* out) {
    if (!text) return 0;
    if (!strcmp(text, "int8")) *out = VX_DTYPE_I8;
    else if (!strcmp(text, "uint8")) *out = VX_DTYPE_U8;
    else if (!strcmp(text, "float32")) *out = VX_DTYPE_F32;
    else return 0;
    return 1;
}

static int object_has_only(const VxjValue* object, const char* const* allowed, size_t allowed_count) {
    if (!object || object->kind != VXJ_OBJECT) return 0;
    for (const VxjValue* m = object->first; m; m = m->next) {
        size_t i = 0;
        while (i < allowed_count && strcmp(allowed[i], m->key)) i++;
        if (i == allowed_count) return 0;
    }
    return 1;
}

/* One descriptor of the central quantization table, resolved to its parameter tensors.
 * per_axis_extent = 0 asks for the per_tensor form. */
static VxStatus resolve_affine(const PackagePlan* plan, const VxjValue* table, const char* target,
                               VxDataType target_dtype, uint32_t target_rank, int64_t per_axis_extent,
                               VxstTensor* scale, VxstTensor* zero_point, Failure* failure) {
    static const char* const tensor_fields[] = {"scheme", "scale_tensor", "zero_point_tensor"};
    static const char* const axis_fields[] = {"scheme", "axis", "scale_tensor", "zero_point_tensor"};
    const VxjValue* d = vxj_member(table, target);
    const char* scheme = vxj_member_string(d, "scheme");
    const char* scale_name = vxj_member_string(d, "scale_tensor");
    const char* zp_name = vxj_member_string(d, "zero_point_tensor");
    if (!d || !scheme || !scale_name || !zp_name)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "no complete affine descriptor for tensor '%s'", target);
    if (per_axis_extent) {
        const VxjValue* axis = vxj_member(d, "axis");
        int64_t a;
        if (strcmp(scheme, "per_axis") || !object_has_only(d, axis_fields, 4) || !axis || axis->kind != VXJ_NUMBER ||
            !axis->is_integer)
            return refuse(failure, VX_STATUS_INVALID_GRAPH, "tensor '%s' needs a per_axis descriptor", target);
        a = axis->integer < 0 ? axis->integer + (int64_t)target_rank : axis->integer;
        if (a != 0)
            return refuse(failure, VX_STATUS_BACKEND_UNSUPPORTED,
                          "weight '%s' must be quantized per output channel (axis 0)", target);
    } else if (strcmp(scheme, "per_tensor") || !object_has_only(d, tensor_fields, 3)) {
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "tensor '%s' needs a per_tensor descriptor", target);
    }
    if (!strcmp(scale_name, zp_name))
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "scale and zero point of '%s' name the same tensor", target);
    if (vxj_member(table, scale_name) || vxj_member(table, zp_name))
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "a quantization parameter of '%s' is itself quantized", target);
    if (find_tensor(plan, scale_name, scale) != 1 || find_tensor(plan, zp_name, zero_point) != 1)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "quantization parameters of '%s' do not resolve uniquely",
                      target);
    const int64_t want = per_axis_extent ? per_axis_extent : 1;
    const char* zp_dtype = target_dtype == VX_DTYPE_I8 ? "I8" : "U8";
    if (strcmp(scale->dtype, "F32") || scale->rank != 1 || scale->shape[0] != want || strcmp(zero_point->dtype, zp_dtype) ||
        zero_point->rank != 1 || zero_point->shape[0] != want)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "quantization parameters of '%s' have the wrong dtype or shape",
                      target);
    for (int64_t i = 0; i < want; i++) {
        float s;
        memcpy(&s, scale->data + 4 * i, 4);
        if (!(s > 0.0f) || !isfinite(s))
            return refuse(failure, VX_STATUS_INVALID_GRAPH, "a scale of '%s' is not finite and positive", target);
    }
    return VX_STATUS_OK;
}

static int32_t typed_zero_point(const VxstTensor* t, int64_t index) {
    return !strcmp(t->dtype, "I8") ? (int32_t)((const int8_t*)t->data)[index] : (int32_t)t->data[index];
}

/* The central table of affine descriptors, or NULL (with the refusal filled in). */
static const VxjValue* quantization_table(const VxjValue* root, Failure* failure) {
    static const char* const table_fields[] = {"format", "tensors"};
    const VxjValue* quantization = vxj_member(root, "quantization");
    const VxjValue* table = vxj_member(quantization, "tensors");
    const char* table_format = vxj_member_string(quantization, "format");
    if (!quantization || !object_has_only(quantization, table_fields, 2) || !table_format ||
        strcmp(table_format, "volvox-affine-safetensors/v1") || !table || table->kind != VXJ_OBJECT || !table->count) {
        refuse(failure, VX_STATUS_INVALID_GRAPH, "graph has no volvox-affine-safetensors/v1 quantization table%s", "");
        return NULL;
    }
    return table;
}

/* QuantizeLinear (float32 -> int8/uint8) or DequantizeLinear (the reverse) with per-tensor
 * parameters.  The node names its scale and zero point, and the table's descriptor of the byte
 * tensor must name the same two tensors. */
static VxStatus plan_boundary(PackagePlan* plan, const VxjValue* root, const VxjValue* node, int quantize,
                              Failure* failure) {
    const VxjValue* node_inputs = vxj_member(node, "inputs");
    const char* scale_name = vxj_member_string(node_inputs, "scale");
    const char* zp_name = vxj_member_string(node_inputs, "zero_point");
    const char* byte_name = quantize ? plan->output_name : plan->input_name;
    const VxDataType byte_dtype = quantize ? plan->output_dtype : plan->input_dtype;
    const VxDataType real_dtype = quantize ? plan->input_dtype : plan->output_dtype;
    const VxjValue* table = quantization_table(root, failure);
    const VxjValue* descriptor;
    VxstTensor scale, zero_point;
    VxStatus status;
    if (!table) return failure->status;
    if (!scale_name || !zp_name)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "node '%s' names no scale or zero point", plan->node_id);
    if (real_dtype != VX_DTYPE_F32 || byte_dtype == VX_DTYPE_F32 || plan->d_in != plan->d_out)
        return refuse(failure, VX_STATUS_INVALID_GRAPH,
                      "node '%s' must convert between float32 and int8/uint8 of one shape", plan->node_id);
    status = resolve_affine(plan, table, byte_name, byte_dtype, 2, 0, &scale, &zero_point, failure);
    if (status != VX_STATUS_OK) return status;
    descriptor = vxj_member(table, byte_name);
    if (strcmp(vxj_member_string(descriptor, "scale_tensor"), scale_name) ||
        strcmp(vxj_member_string(descriptor, "zero_point_tensor"), zp_name))
        return refuse(failure, VX_STATUS_INVALID_GRAPH,
                      "node '%s' and the quantization table name different parameters", plan->node_id);
    memcpy(&plan->boundary_scale, scale.data, 4);
    plan->boundary_zero_point = typed_zero_point(&zero_point, 0);
    plan->kind = quantize ? PLAN_QUANTIZE : PLAN_DEQUANTIZE;
    return VX_STATUS_OK;
}

/* RequantizeLinear: int8/uint8 -> int8/uint8 between the central per-tensor descriptors of its input
 * and its output; the node itself names no parameter tensors
 * (native/src/runtime/engine_runtime_w8a8.inc:3470-3481). */
static VxStatus plan_requantize(PackagePlan* plan, const VxjValue* root, Failure* failure) {
    const VxjValue* table = quantization_table(root, failure);
    VxstTensor scale, zero_point;
    VxStatus status;
    if (!table) return failure->status;
    if (plan->input_dtype == VX_DTYPE_F32 || plan->output_dtype == VX_DTYPE_F32 || plan->d_in != plan->d_out)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "node '%s' must convert between int8/uint8 tensors of one shape",
                      plan->node_id);
    status = resolve_affine(plan, table, plan->input_name, plan->input_dtype, 2, 0, &scale, &zero_point, failure);
    if (status != VX_STATUS_OK) return status;
    memcpy(&plan->input_scale, scale.data, 4);
    plan->input_zero_point = typed_zero_point(&zero_point, 0);
    status = resolve_affine(plan, table, plan->output_name, plan->output_dtype, 2, 0, &scale, &zero_point, failure);
    if (status != VX_STATUS_OK) return status;
    memcpy(&plan->output_scale, scale.data, 4);
    plan->output_zero_point = typed_zero_point(&zero_point, 0);
    {
        /* the operator's own contract: the ratio of the scales is a positive finite f32 */
        volatile float multiplier = plan->input_scale / plan->output_scale;
        if (!(multiplier > 0.0f) || !isfinite(multiplier))
            return refuse(failure, VX_STATUS_INVALID_GRAPH, "the scales of node '%s' have no finite positive ratio",
                          plan->node_id);
    }
    plan->kind = PLAN_REQUANTIZE;
    return VX_STATUS_OK;
}

/* An aligned copy of `bytes` payload bytes, owned by the plan; NULL when memory runs out. */
static const void* aligned_payload(PackagePlan* plan, const void* data, size_t bytes) {
    void* copy;
    if (plan->aligned_count == sizeof(plan->aligned_copies) / sizeof(plan->aligned_copies[0])) return NULL;
    copy = malloc(bytes ? bytes : 1);
    if (!copy) return NULL;
    memcpy(copy, data, bytes);
    plan->aligned_copies[plan->aligned_count++] = copy;
    return copy;
}

static VxStatus plan_qlinear(PackagePlan* plan, const VxjValue* root, const VxjValue* node, Failure* failure) {
    const VxjValue* node_inputs = vxj_member(node, "inputs");
    const char* weight_name = vxj_member_string(node_inputs, "weight");
    const char* bias_name = vxj_member_string(node_inputs, "bias");
    const VxjValue* table = quantization_table(root, failure);
    VxstTensor weight, bias, scale, zero_point;
    VxStatus status;
    if (!table) return failure->status;
    if (!weight_name) return refuse(failure, VX_STATUS_INVALID_GRAPH, "QLinear node '%s' names no weight", plan->node_id);
    if (plan->input_dtype == VX_DTYPE_F32 || plan->output_dtype == VX_DTYPE_F32)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "QLinear node '%s' needs int8/uint8 input and output",
                      plan->node_id);
    if (find_tensor(plan, weight_name, &weight) != 1)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "weight '%s' does not resolve uniquely", weight_name);
    if ((strcmp(weight.dtype, "I8") && strcmp(weight.dtype, "U8")) || weight.rank != 2 ||
        weight.shape[0] != (int64_t)plan->d_out || weight.shape[1] != (int64_t)plan->d_in)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "weight '%s' is not I8/U8 [d_out, d_in]", weight_name);
    plan->weight = weight.data;
    plan->weight_dtype = !strcmp(weight.dtype, "I8") ? VXHIP_DTYPE_I8 : VXHIP_DTYPE_U8;

    status = resolve_affine(plan, table, plan->input_name, plan->input_dtype, 2, 0, &scale, &zero_point, failure);
    if (status != VX_STATUS_OK) return status;
    memcpy(&plan->input_scale, scale.data, 4);
    plan->input_zero_point = typed_zero_point(&zero_point, 0);

    status = resolve_affine(plan, table, plan->output_name, plan->output_dtype, 2, 0, &scale, &zero_point, failure);
    if (status != VX_STATUS_OK) return status;
    memcpy(&plan->output_scale, scale.data, 4);
    plan->output_zero_point = typed_zero_point(&zero_point, 0);

    status = resolve_affine(plan, table, weight_name, plan->weight_dtype == VXHIP_DTYPE_I8 ? VX_DTYPE_I8 : VX_DTYPE_U8,
                            2, plan->d_out, &scale, &zero_point, failure);
    if (status != VX_STATUS_OK) return status;
    plan->weight_scales = (const float*)aligned_payload(plan, scale.data, sizeof(float) * plan->d_out);
    plan->weight_zero_points = (int32_t*)malloc(sizeof(int32_t) * plan->d_out);
    if (!plan->weight_scales || !plan->weight_zero_points) return refuse(failure, VX_STATUS_OUT_OF_MEMORY, "out of memory%s", "");
    for (uint32_t n = 0; n < plan->d_out; n++) plan->weight_zero_points[n] = typed_zero_point(&zero_point, n);

    if (bias_name) {
        if (find_tensor(plan, bias_name, &bias) != 1 || strcmp(bias.dtype, "I32") || bias.rank != 1 ||
            bias.shape[0] != (int64_t)plan->d_out)
            return refuse(failure, VX_STATUS_INVALID_GRAPH, "bias '%s' is not a unique I32 [d_out] tensor", bias_name);
        plan->bias_i32 = (const int32_t*)aligned_payload(plan, bias.data, sizeof(int32_t) * plan->d_out);
        if (!plan->bias_i32) return refuse(failure, VX_STATUS_OUT_OF_MEMORY, "out of memory%s", "");
    }
    plan->kind = PLAN_QLINEAR;
    return VX_STATUS_OK;
}

static VxStatus plan_packed(PackagePlan* plan, const VxjValue* node, VxPackedArithmetic arithmetic,
                            Failure* failure) {
    const VxjValue* node_inputs = vxj_member(node, "inputs");
    const VxjValue* params = vxj_member(node, "params");
    const VxjValue* group = vxj_member(params, "group_size");
    const VxjValue* bits = vxj_member(params, "weight_bits");
    const char* weight_name = vxj_member_string(node_inputs, "weight");
    const char* scale_name = vxj_member_string(node_inputs, "scale");
    const char* bias_name = vxj_member_string(node_inputs, "bias");
    VxstTensor weight, scale, bias;
    if (arithmetic != VX_PACKED_ARITHMETIC_DYNAMIC_I8)
        return refuse(failure, VX_STATUS_BACKEND_UNSUPPORTED,
                      "PackedLinear is offered under DYNAMIC_I8 packed arithmetic only%s", "");
    if (!group || group->kind != VXJ_NUMBER || !group->is_integer || !bits || bits->kind != VXJ_NUMBER ||
        !bits->is_integer || !weight_name || !scale_name)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "PackedLinear node '%s' lacks weight, scale or parameters",
                      plan->node_id);
    if (bits->integer != 8 && bits->integer != 4 && bits->integer != 3 && bits->integer != 2)
        return refuse(failure, VX_STATUS_BACKEND_UNSUPPORTED,
                      "PackedLinear node '%s': weight_bits must be 2, 3, 4 or 8", plan->node_id);
    if (group->integer != 32 && group->integer != 64 && group->integer != 128 && group->integer != 256)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "PackedLinear node '%s': group_size must be 32, 64, 128 or 256",
                      plan->node_id);
    if (plan->input_dtype != VX_DTYPE_F32 || plan->output_dtype != VX_DTYPE_F32)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "PackedLinear node '%s' needs float32 input and output",
                      plan->node_id);
    plan->group_size = (uint32_t)group->integer;
    plan->weight_bits = (uint32_t)bits->integer;
    /* vx_packed_words (src/kernels/packed_linear_ops.inc:246-248) */
    const int64_t words = ((int64_t)plan->d_in / 32) * bits->integer + (((int64_t)plan->d_in % 32) * bits->integer + 31) / 32;
    const int64_t groups = ((int64_t)plan->d_in + plan->group_size - 1) / plan->group_size;
    if (find_tensor(plan, weight_name, &weight) != 1 || (strcmp(weight.dtype, "I32") && strcmp(weight.dtype, "U32")) ||
        weight.rank != 2 || weight.shape[0] != (int64_t)plan->d_out || weight.shape[1] != words)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "packed weight '%s' is not I32 [d_out, words(d_in, weight_bits)]",
                      weight_name);
    if (find_tensor(plan, scale_name, &scale) != 1 || strcmp(scale.dtype, "F32") || scale.rank != 2 ||
        scale.shape[0] != (int64_t)plan->d_out || scale.shape[1] != groups)
        return refuse(failure, VX_STATUS_INVALID_GRAPH, "group scales '%s' are not F32 [d_out, groups]", scale_name);
    /* (the packed words are only ever copied bytewise to the device; they stay in the mapping) */
    plan->packed_words = (const uint32_t*)(const void*)weight.data;
    plan->group_scales = (const float*)aligned_payload(plan, scale.data, sizeof(float) * (size_t)plan->d_out * (size_t)groups);
    if (!plan->group_scales) return refuse(failure, VX_STATUS_OUT_OF_MEMORY, "out of memory%s", "");
    if (bias_name) {
        if (find_tensor(plan, bias_name, &bias) != 1 || strcmp(bias.dtype, "F32") || bias.rank != 1 ||
            bias.shape[0] != (int64_t)plan->d_out)
            return refuse(failure, VX_STATUS_INVALID_GRAPH, "bias '%s' is not a unique F32 [d_out] tensor", bias_name);
        plan->bias_f32 = (const float*)aligned_payload(plan, bias.data, sizeof(float) * plan->d_out);
        if (!plan->bias_f32) return refuse(failure, VX_STATUS_OUT_OF_MEMORY, "out of memory%s", "");
    }
    plan->kind = PLAN_PACKED_LINEAR;
    return VX_STATUS_OK;
}

/* A positive extent that fits the kernels' 32-bit row lengths, else 0. */
static uint32_t fixed_extent(const VxjValue* v) {
    return v && v->kind == VXJ_NUMBER && v->is_integer && v->integer > 0 && v->integer <= INT32_MAX
               ? (uint32_t)v->integer : 0u;
}

/* Two declared extents are the same number or the same symbol. */
static int same_extent(const VxjValue* a, const VxjValue* b) {
    if (!a || !b || a->kind != b->kind) return 0;
    if (a->kind == VXJ_NUMBER) return a->is_integer && b->is_integer && a->integer == b->integer;
    return a->kind == VXJ_STRING && !strcmp(a->string, b->string);
}

/* Reads graph.json and the weight files named by the model source into a chain of node plans. */
static VxStatus plan_package(const VxModelSource* source, VxPackedArithmetic arithmetic, ChainPlan* chain,
                             Failure* failure) {
    size_t length = 0;
    const char* json_error = NULL;
    char* text;
    VxjValue* root;
    VxStatus status = VX_STATUS_OK;
    memset(chain, 0, sizeof(*chain));
    text = read_text_file(source->graph_path, &length);
    if (!text) return refuse(failure, VX_STATUS_IO_ERROR, "cannot read graph document '%s'", source->graph_path);
    root = vxj_parse(text, length, &json_error);
    free(text);
    if (!root) return refuse(failure, VX_STATUS_INVALID_GRAPH, "graph document is not valid JSON: %s", json_error);

    do {
        const char* format = vxj_member_string(root, "format");
        const VxjValue* inputs = vxj_member(root, "inputs");
        const VxjValue* nodes = vxj_member(root, "nodes");
        const VxjValue* outputs = vxj_member(root, "outputs");
        const VxjValue* first_input = inputs && inputs->kind == VXJ_OBJECT ? inputs->first : NULL;
        const VxjValue* in_shape = vxj_member(first_input, "shape");
        if (!format || strcmp(format, "volvox-graph/v1")) {
            status = refuse(failure, VX_STATUS_INVALID_GRAPH, "graph format is not volvox-graph/v1%s", "");
            break;
        }
        /* representations v1 retired: an artifact that carries one is not a v1 package
         * (docs/w8a8-safetensors.md:176-188) */
        if (vxj_member(root, "weights_quantization") || vxj_member(root, "weights_quantization_storage")) {
            status = refuse(failure, VX_STATUS_INVALID_GRAPH,
                            "the graph carries a retired quantization field (weights_quantization, "
                            "weights_quantization_storage or an inline input quantization)%s", "");
            break;
        }
        for (const VxjValue* in = first_input; in; in = in->next)
            if (in->kind == VXJ_OBJECT && vxj_member(in, "quantization")) {
                status = refuse(failure, VX_STATUS_INVALID_GRAPH,
                                "the graph carries a retired quantization field (weights_quantization, "
                                "weights_quantization_storage or an inline input quantization)%s", "");
                break;
            }
        if (status != VX_STATUS_OK) break;
        if (!nodes || nodes->kind != VXJ_ARRAY || !nodes->count || nodes->count > MAX_CHAIN_NODES || !inputs ||
            inputs->kind != VXJ_OBJECT || !inputs->count || inputs->count > MAX_GRAPH_PORTS || !outputs ||
            outputs->kind != VXJ_ARRAY || !outputs->count || outputs->count > MAX_GRAPH_PORTS) {
            status = refuse(failure, VX_STATUS_BACKEND_UNSUPPORTED,
                            "this provider compiles graphs of up to 64 nodes with up to 8 inputs and 8 outputs%s", "");
            break;
        }
        if (!in_shape || in_shape->kind != VXJ_ARRAY || !in_shape->count) {
            status = refuse(failure, VX_STATUS_INVALID_GRAPH, "graph input or output declaration is incomplete%s", "");
            break;
        }
        /* the graph inputs: dense on the last axis (that extent is a number in every declaration),
         * one set of leading extents -- the rows -- for all of them */
        for (const VxjValue* in = first_input; in && status == VX_STATUS_OK; in = in->next) {
            PlanTensor* t = &chain->tensors[chain->tensor_count];
            const VxjValue* shape = vxj_member(in, "shape");
            if (!copy_name(t->name, in->key) || !graph_dtype(vxj_member_string(in, "dtype"), &t->dtype) || !shape ||
                shape->kind != VXJ_ARRAY || shape->count != in_shape->count) {
                status = refuse(failure, VX_STATUS_INVALID_GRAPH, "graph input or output declaration is incomplete%s", "");
                break;
            }
            for (size_t axis = 0; axis + 1 < in_shape->count; axis++)
                if (!same_extent(vxj_item(in_shape, axis), vxj_item(shape, axis)))
                    status = refuse(failure, VX_STATUS_BACKEND_UNSUPPORTED,
                                    "graph input '%s' does not share the leading extents of the first input", t->name);
            t->d = fixed_extent(vxj_item(shape, shape->count - 1));
            if (status == VX_STATUS_OK && !t->d)
                status = refuse(failure, VX_STATUS_INVALID_GRAPH, "the input's last extent must be a fixed d_in%s", "");
            chain->input_slots[chain->input_count++] = (uint32_t)chain->tensor_count++;
        }
        if (status != VX_STATUS_OK) break;
        memcpy(chain->input_name, chain->tensors[0].name, sizeof(chain->input_name));
        chain->input_dtype = chain->tensors[0].dtype;
        chain->d_in = chain->tensors[0].d;
        chain->files = (VxstFile**)calloc(source->weight_path_count ? source->weight_path_count : 1, sizeof(VxstFile*));
        chain->nodes = (PackagePlan*)calloc(nodes->count, sizeof(PackagePlan));
        if (!chain->files || !chain->nodes) {
            status = refuse(failure, VX_STATUS_OUT_OF_MEMORY, "out of memory%s", "");
            break;
        }
        for (size_t i = 0; i < source->weight_path_count && status == VX_STATUS_OK; i++) {
            char error[VX_REPORT_MESSAGE_CAPACITY];
            if (vxst_open(source->weight_paths[i], &chain->files[chain->file_count], error, sizeof(error)) != 0) {
                status = refuse(failure, VX_STATUS_IO_ERROR, "%s", error);
            } else {
                const VxstFile* opened = chain->files[chain->file_count++];
                /* SafeTensors metadata is no quantization authority, and the retired keys make the
                 * file invalid (docs/w8a8-safetensors.md:100-102) */
                if (vxst_metadata_has(opened, "weights_quantization") ||
                    vxst_metadata_has(opened, "weights_quantization_storage"))
                    status = refuse(failure, VX_STATUS_INVALID_GRAPH,
                                    "weight file '%s' carries retired quantization metadata", source->weight_paths[i]);
            }
        }
        if (status != VX_STATUS_OK) break;

        for (const VxjValue* node = nodes->first; node && status == VX_STATUS_OK; node = node->next) {
            PackagePlan* plan = &chain->nodes[chain->count];
            const char* op = vxj_member_string(node, "opType");
            const VxjValue* out = vxj_member(vxj_member(node, "outputs"), "out");
            const VxjValue* out_shape = vxj_member(out, "shape");
            const char* fed = vxj_member_string(vxj_member(node, "inputs"), "input");
            PlanTensor* written = &chain->tensors[chain->tensor_count];
            size_t reads = chain->tensor_count;
            chain->count++;
            if (node->kind == VXJ_OBJECT && vxj_member(node, "outputs_quantization")) {
                status = refuse(failure, VX_STATUS_INVALID_GRAPH,
                                "a node carries the retired outputs_quantization field%s", "");
                break;
            }
            plan->files = chain->files;
            plan->file_count = chain->file_count;
            if (!op || !out || !copy_name(plan->node_id, vxj_member_string(node, "id")) ||
                !copy_name(plan->output_name, vxj_member_string(out, "tensor")) ||
                !graph_dtype(vxj_member_string(out, "dtype"), &plan->output_dtype) || !out_shape ||
                out_shape->kind != VXJ_ARRAY || out_shape->count != in_shape->count) {
                status = refuse(failure, VX_STATUS_INVALID_GRAPH, "node or tensor declaration is incomplete%s", "");
                break;
            }
            /* a node reads a graph input or what an earlier node wrote, and writes a new tensor */
            for (size_t t = 0; fed && t < chain->tensor_count; t++)
                if (!strcmp(chain->tensors[t].name, fed)) reads = t;
            if (reads == chain->tensor_count) {
                status = refuse(failure, VX_STATUS_INVALID_GRAPH,
                                "node '%s' reads a tensor that neither a graph input nor an earlier node provides",
                                plan->node_id);
                break;
            }
            for (size_t t = 0; t < chain->tensor_count; t++)
                if (!strcmp(chain->tensors[t].name, plan->output_name))
                    status = refuse(failure, VX_STATUS_INVALID_GRAPH, "node '%s' writes a tensor that already exists",
                                    plan->node_id);
            /* rows pass through unchanged: the leading extents are the graph input's */
            for (size_t axis = 0; axis + 1 < in_shape->count && status == VX_STATUS_OK; axis++)
                if (!same_extent(vxj_item(in_shape, axis), vxj_item(out_shape, axis)))
                    status = refuse(failure, VX_STATUS_INVALID_GRAPH,
                                    "node '%s' changes a leading extent", plan->node_id);
            if (status != VX_STATUS_OK) break;
            memcpy(plan->input_name, chain->tensors[reads].name, sizeof(plan->input_name));
            plan->input_dtype = chain->tensors[reads].dtype;
            plan->d_in = chain->tensors[reads].d;
            plan->input_slot = (uint32_t)reads;
            plan->output_slot = (uint32_t)chain->tensor_count;
            plan->d_out = fixed_extent(vxj_item(out_shape, out_shape->count - 1));
            if (!plan->d_out) {
                status = refuse(failure, VX_STATUS_INVALID_GRAPH, "the last extent of '%s' must be fixed",
                                plan->output_name);
                break;
            }
            if (!strcmp(op, "QLinear") || !strcmp(op, "QGemm") || !strcmp(op, "QMatMul"))
                status = plan_qlinear(plan, root, node, failure);
            else if (!strcmp(op, "PackedLinear"))
                status = plan_packed(plan, node, arithmetic, failure);
            else if (!strcmp(op, "QuantizeLinear") || !strcmp(op, "DequantizeLinear"))
                status = plan_boundary(plan, root, node, op[0] == 'Q', failure);
            else if (!strcmp(op, "RequantizeLinear"))
                status = plan_requantize(plan, root, failure);
            else
                status = refuse(failure, VX_STATUS_BACKEND_UNSUPPORTED, "operator '%s' is not offered by this provider",
                                op);
            if (plan->kind == PLAN_PACKED_LINEAR) chain->any_packed = 1;
            memcpy(written->name, plan->output_name, sizeof(written->name));
            written->dtype = plan->output_dtype;
            written->d = plan->d_out;
            chain->tensor_count++;
        }
        if (status != VX_STATUS_OK) break;
        /* the graph outputs: distinct tensors written by nodes */
        for (const VxjValue* o = outputs->first; o && status == VX_STATUS_OK; o = o->next) {
            size_t slot = chain->tensor_count;
            for (size_t t = chain->input_count; o->kind == VXJ_STRING && t < chain->tensor_count; t++)
                if (!strcmp(chain->tensors[t].name, o->string)) slot = t;
            for (size_t k = 0; k < chain->output_count; k++)
                if (chain->output_slots[k] == slot) slot = chain->tensor_count;
            if (slot == chain->tensor_count) {
                status = refuse(failure, VX_STATUS_INVALID_GRAPH, "no node writes the graph output '%s' (or it is listed twice)",
                                o->kind == VXJ_STRING ? o->string : "(not a name)");
                break;
            }
            chain->output_slots[chain->output_count++] = (uint32_t)slot;
        }
        if (status != VX_STATUS_OK) break;
        memcpy(chain->output_name, chain->tensors[chain->output_slots[0]].name, sizeof(chain->output_name));
        chain->output_dtype = chain->tensors[chain->output_slots[0]].dtype;
        chain->d_out = chain->tensors[chain->output_slots[0]].d;
    } while (0);
    vxj_free(root);
    if (status != VX_STATUS_OK) chain_release(chain);
    return status;
}

#include "decoder_route.inc"

/* ---- SPI callbacks ---------------------------------------------------------------- */

static VxStatus hip_runtime_create(void* user_data, const VxRuntimeOptions* options, void** out_runtime,
                                   VxReport* report) {
    HipRuntime* runtime;
    (void)user_data;
    if (!out_runtime) return VX_STATUS_INVALID_ARGUMENT;
    *out_runtime = NULL;
    if (!options || options->struct_size != sizeof(*options)) return VX_STATUS_INVALID_ARGUMENT;
    if (vxhip_device_count() <= 0) {
        /* optional hardware absent: the runtime omits this provider (runtime/backend_sdk.c:206-213) */
        fill_report(report, NULL, VX_STATUS_BACKEND_UNAVAILABLE, VX_STAGE_RUNTIME_CREATE, VX_CODE_BACKEND_UNAVAILABLE,
                    "no gfx950 device is visible");
        return VX_STATUS_BACKEND_UNAVAILABLE;
    }
    runtime = (HipRuntime*)calloc(1, sizeof(*runtime));
    if (!runtime) return VX_STATUS_OUT_OF_MEMORY;
    runtime->device = 0;
    if (vxhip_device_name(0, runtime->device_name, sizeof(runtime->device_name)) != VXHIP_OK)
        snprintf(runtime->device_name, sizeof(runtime->device_name), "%s", "gfx950");
    *out_runtime = runtime;
    fill_report(report, runtime, VX_STATUS_OK, VX_STAGE_RUNTIME_CREATE, VX_CODE_NONE, "hip-gfx950 runtime created");
    return VX_STATUS_OK;
}

static void hip_runtime_destroy(void* runtime_instance) {
    free(runtime_instance);
}

static int policy_names(const VxBackendPolicy* policy, const char* name) {
    if (!policy || policy->struct_size != sizeof(*policy) || !policy->backends) return 0;
    for (size_t i = 0; i < policy->backend_count; i++)
        if (policy->backends[i] && !strcmp(policy->backends[i], name)) return 1;
    return 0;
}

static void hip_compiled_destroy(void* compiled_instance) {
    HipCompiled* compiled = (HipCompiled*)compiled_instance;
    if (!compiled) return;
    decoder_model_release(compiled->decoder);
    for (size_t i = 0; i < compiled->stage_count; i++) {
        if (compiled->stages[i].qlinear) vxhip_qlinear_destroy(compiled->stages[i].qlinear);
        if (compiled->stages[i].packed) vxhip_packed_linear_destroy(compiled->stages[i].packed);
    }
    free(compiled->stages);
    free(compiled);
}

/* The logical specifications the core hands over must describe the same tensors as the graph:
 * every graph input and output by name, with its element type, a fixed last extent and one common
 * set of leading dimensions. */
static const VxTensorSpec* spec_named(const VxTensorSpec* specs, size_t count, const char* name) {
    for (size_t i = 0; specs && i < count; i++)
        if (specs[i].struct_size == sizeof(specs[i]) && specs[i].name && !strcmp(specs[i].name, name)) return &specs[i];
    return NULL;
}

static int specs_match(const VxBackendCompileInput* input, const ChainPlan* plan, HipCompiled* compiled) {
    const VxTensorSpec* first = spec_named(input->inputs, input->input_count, plan->tensors[plan->input_slots[0]].name);
    int symbolic_rows = 1;
    if (input->input_count != plan->input_count || input->output_count != plan->output_count || !first ||
        first->rank < 1 || first->rank > VX_MAX_TENSOR_RANK)
        return 0;
    compiled->rank = first->rank;
    for (size_t k = 0; k < plan->input_count + plan->output_count; k++) {
        const int is_input = k < plan->input_count;
        const PlanTensor* t = &plan->tensors[is_input ? plan->input_slots[k] : plan->output_slots[k - plan->input_count]];
        const VxTensorSpec* spec = is_input ? spec_named(input->inputs, input->input_count, t->name)
                                            : spec_named(input->outputs, input->output_count, t->name);
        const VxDimensionConstraint* last;
        if (!spec || spec->dtype != t->dtype || spec->rank != first->rank || spec->location != VX_MEMORY_HOST) return 0;
        last = &spec->dimensions[spec->rank - 1];
        if (last->kind != VX_DIMENSION_FIXED || last->min != (int64_t)t->d || last->max != last->min) return 0;
        for (uint32_t axis = 0; axis + 1 < first->rank; axis++) {
            const VxDimensionConstraint* a = &first->dimensions[axis];
            const VxDimensionConstraint* b = &spec->dimensions[axis];
            if (a->min < 1 || a->max < a->min || a->multiple_of < 1 || a->min != b->min || a->max != b->max ||
                a->multiple_of != b->multiple_of)
                return 0;
        }
        if (spec->dimensions[0].kind != VX_DIMENSION_SYMBOLIC) symbolic_rows = 0;
    }
    for (uint32_t axis = 0; axis + 1 < first->rank; axis++) {
        compiled->lead_min[axis] = first->dimensions[axis].min;
        compiled->lead_max[axis] = first->dimensions[axis].max;
        compiled->lead_multiple[axis] = first->dimensions[axis].multiple_of;
    }
    compiled->batch_capable = first->rank >= 2 && symbolic_rows && first->dimensions[0].min <= 1 &&
                              first->dimensions[0].multiple_of == 1 && input->independent_batch_proof_protocol &&
                              !strcmp(input->independent_batch_proof_protocol,
                                      VX_BACKEND_INDEPENDENT_BATCH_PROOF_PROTOCOL) &&
                              input->independent_batch_proof_identity &&
                              strlen(input->independent_batch_proof_identity) < sizeof(compiled->batch_proof_identity) &&
                              strlen(input->graph_fingerprint) < sizeof(compiled->graph_fingerprint);
    if (compiled->batch_capable) {
        snprintf(compiled->graph_fingerprint, sizeof(compiled->graph_fingerprint), "%s", input->graph_fingerprint);
        snprintf(compiled->batch_proof_identity, sizeof(compiled->batch_proof_identity), "%s",
                 input->independent_batch_proof_identity);
    }
    return 1;
}

/* A graph whose first node is an Embedding is a decoder graph: read it, open the weight files and
 * compile the decoder route.  *is_decoder = 0 leaves everything to the chain reader. */
static VxStatus try_decoder(const VxModelSource* source, VxPackedArithmetic arithmetic, int32_t device, int* is_decoder,
                            DecoderModel** out, Failure* failure) {
    size_t length = 0, opened = 0;
    const char* json_error = NULL;
    char* text = read_text_file(source->graph_path, &length);
    VxjValue* root;
    VxstFile** files;
    VxStatus status = VX_STATUS_OK;
    *is_decoder = 0;
    *out = NULL;
    if (!text) return VX_STATUS_OK; /* the chain reader reports what is wrong with the document */
    root = vxj_parse(text, length, &json_error);
    free(text);
    if (!root) return VX_STATUS_OK;
    if (!graph_is_decoder(root)) {
        vxj_free(root);
        return VX_STATUS_OK;
    }
    *is_decoder = 1;
    files = (VxstFile**)calloc(source->weight_path_count ? source->weight_path_count : 1, sizeof(VxstFile*));
    if (!files) status = refuse(failure, VX_STATUS_OUT_OF_MEMORY, "out of memory%s", "");
    {
        const char* format = vxj_member_string(root, "format");
        if (status == VX_STATUS_OK && (!format || strcmp(format, "volvox-graph/v1")))
            status = refuse(failure, VX_STATUS_INVALID_GRAPH, "graph format is not volvox-graph/v1%s", "");
    }
    for (size_t i = 0; i < source->weight_path_count && status == VX_STATUS_OK; i++) {
        char error[VX_REPORT_MESSAGE_CAPACITY];
        if (vxst_open(source->weight_paths[i], &files[opened], error, sizeof(error)) != 0)
            status = refuse(failure, VX_STATUS_IO_ERROR, "%s", error);
        else
            opened++;
    }
    if (status == VX_STATUS_OK) status = decoder_compile(root, files, opened, device, arithmetic, out, failure);
    for (size_t i = 0; i < opened; i++) vxst_close(files[i]);
    free(files);
    vxj_free(root);
    return status;
}

/* The logical specifications of a decoder graph: the id rows in, ids and/or logits out. */
static int decoder_specs_match(const VxBackendCompileInput* input, const DecoderModel* m) {
    const size_t want_outputs = (size_t)(m->publish_ids + m->publish_logits);
    const VxTensorSpec* in;
    if (input->input_count != 1 || input->output_count != want_outputs || !input->inputs || !input->outputs) return 0;
    in = &input->inputs[0];
    if (in->struct_size != sizeof(*in) || !in->name || strcmp(in->name, m->input_name) || in->dtype != VX_DTYPE_I32 ||
        in->rank != 2 || in->location != VX_MEMORY_HOST || in->dimensions[0].kind != VX_DIMENSION_FIXED ||
        in->dimensions[0].min != (int64_t)m->slots || in->dimensions[1].kind != VX_DIMENSION_FIXED ||
        in->dimensions[1].min != (int64_t)m->capacity)
        return 0;
    for (size_t i = 0; i < input->output_count; i++) {
        const VxTensorSpec* o = &input->outputs[i];
        if (o->struct_size != sizeof(*o) || !o->name || o->location != VX_MEMORY_HOST) return 0;
        if (m->publish_ids && !strcmp(o->name, m->ids_name)) {
            if (o->dtype != VX_DTYPE_I32 || o->rank != 1 || o->dimensions[0].min != (int64_t)m->slots) return 0;
        } else if (m->publish_logits && !strcmp(o->name, m->logits_name)) {
            if (o->dtype != VX_DTYPE_F32 || o->rank != 2 || o->dimensions[0].min != (int64_t)m->slots ||
                o->dimensions[1].min != (int64_t)m->vocab)
                return 0;
        } else {
            return 0;
        }
    }
    return 1;
}

static VxStatus hip_compile(void* runtime_instance, const VxBackendCompileInput* input, const VxBackendPolicy* policy,
                            void** out_compiled, VxBackendShapeDomainAttestation* attestation, VxReport* report) {
    HipRuntime* runtime = (HipRuntime*)runtime_instance;
    ChainPlan plan;
    Failure failure = {VX_STATUS_OK, {0}};
    HipCompiled* compiled;
    VxStatus status;
    uint64_t rows_max = 1, resident = 0;
    size_t route_used = 0;
    if (!runtime || !input || input->struct_size != sizeof(*input) || !input->source ||
        input->source->struct_size != sizeof(*input->source) || !input->graph_fingerprint ||
        !input->shape_domain_proof_identity || !out_compiled || !attestation ||
        attestation->struct_size != sizeof(*attestation) || !policy_names(policy, PROVIDER_NAME))
        return VX_STATUS_INVALID_ARGUMENT;
    *out_compiled = NULL;
    if (input->packed_arithmetic == VX_PACKED_ARITHMETIC_DYNAMIC_I4) {
        /* a known option this provider has no executable for: refuse before allocating anything
         * (native/tests/test_packed_arithmetic.inc:111-123) */
        fill_report(report, runtime, VX_STATUS_BACKEND_UNSUPPORTED, VX_STAGE_COMPILE, VX_CODE_BACKEND_UNSUPPORTED,
                    "DYNAMIC_I4 packed arithmetic is not offered");
        return VX_STATUS_BACKEND_UNSUPPORTED;
    }
    {
        /* decoder graphs take their own route (decoder_route.inc) */
        int is_decoder = 0;
        DecoderModel* decoder = NULL;
        status = try_decoder(input->source, input->packed_arithmetic, runtime->device, &is_decoder, &decoder, &failure);
        if (is_decoder) {
            char route[64];
            if (status != VX_STATUS_OK) {
                fill_report(report, runtime, status, VX_STAGE_COMPILE, code_for(status), failure.message);
                return status;
            }
            if (!decoder_specs_match(input, decoder)) {
                decoder_model_release(decoder);
                fill_report(report, runtime, VX_STATUS_INVALID_ARGUMENT, VX_STAGE_COMPILE, VX_CODE_INVALID_ARGUMENT,
                            "logical tensor specifications do not describe the decoder's ids and outputs");
                return VX_STATUS_INVALID_ARGUMENT;
            }
            compiled = (HipCompiled*)calloc(1, sizeof(*compiled));
            if (!compiled) {
                decoder_model_release(decoder);
                return VX_STATUS_OUT_OF_MEMORY;
            }
            compiled->runtime = runtime;
            compiled->decoder = decoder;
            snprintf(compiled->route, sizeof(compiled->route), "hip.decoder.w8a8-packed-linear.layers%u", decoder->layers);
            attestation->graph_fingerprint = input->graph_fingerprint;
            attestation->shape_domain_proof_identity = input->shape_domain_proof_identity;
            {
                const uint64_t rows = (uint64_t)decoder->slots * decoder->capacity;
                const uint64_t kv = (uint64_t)decoder->kv_heads * decoder->head_dim, q = (uint64_t)decoder->q_heads * decoder->head_dim;
                const uint64_t widest = 2u * (uint64_t)decoder->inter > q + 2u * kv ? 2u * (uint64_t)decoder->inter : q + 2u * kv;
                const uint64_t logits = (uint64_t)decoder->slots * decoder->vocab * 4u;
                attestation->maximum_tensor_bytes = rows * widest * 4u > logits ? rows * widest * 4u : logits;
                /* weights; per context the two caches and the work buffers of one full-length call */
                attestation->maximum_resident_bytes =
                    decoder->resident_bytes + 2u * (uint64_t)decoder->layers * rows * kv * 4u +
                    rows * (4u * (uint64_t)decoder->hidden + 3u * q + 2u * kv + 2u * (uint64_t)decoder->inter + 4u) * 4u + 2u * logits;
            }
            attestation->resource_limit_bytes = 0;
            attestation->has_resource_limit = 0;
            attestation->packed_arithmetic = VX_PACKED_ARITHMETIC_DYNAMIC_I8;
            *out_compiled = compiled;
            fill_report(report, runtime, VX_STATUS_OK, VX_STAGE_COMPILE, VX_CODE_NONE, "W8A8 decoder compiled");
            snprintf(route, sizeof(route), "%s", compiled->route);
            attest(report, decoder->node_count, route);
            return VX_STATUS_OK;
        }
    }
    if (!input->input_count || !input->output_count || !input->inputs || !input->outputs) {
        fill_report(report, runtime, VX_STATUS_INVALID_ARGUMENT, VX_STAGE_COMPILE, VX_CODE_INVALID_ARGUMENT,
                    "the compile input names no input or no output");
        return VX_STATUS_INVALID_ARGUMENT;
    }
    status = plan_package(input->source, input->packed_arithmetic, &plan, &failure);
    if (status != VX_STATUS_OK) {
        fill_report(report, runtime, status, VX_STAGE_COMPILE, code_for(status), failure.message);
        return status;
    }
    compiled = (HipCompiled*)calloc(1, sizeof(*compiled));
    if (compiled) compiled->stages = (HipStage*)calloc(plan.count, sizeof(HipStage));
    if (!compiled || !compiled->stages) {
        chain_release(&plan);
        free(compiled);
        return VX_STATUS_OUT_OF_MEMORY;
    }
    if (!specs_match(input, &plan, compiled)) {
        chain_release(&plan);
        hip_compiled_destroy(compiled);
        fill_report(report, runtime, VX_STATUS_INVALID_ARGUMENT, VX_STAGE_COMPILE, VX_CODE_INVALID_ARGUMENT,
                    "logical tensor specifications do not describe the graph's input and output");
        return VX_STATUS_INVALID_ARGUMENT;
    }
    compiled->runtime = runtime;
    memcpy(compiled->tensors, plan.tensors, sizeof(compiled->tensors));
    compiled->tensor_count = plan.tensor_count;
    memcpy(compiled->input_slots, plan.input_slots, sizeof(compiled->input_slots));
    memcpy(compiled->output_slots, plan.output_slots, sizeof(compiled->output_slots));
    compiled->input_count = plan.input_count;
    compiled->output_count = plan.output_count;
    for (size_t t = 0; t < plan.tensor_count; t++) {
        const uint64_t row_bytes = (uint64_t)plan.tensors[t].d * (plan.tensors[t].dtype == VX_DTYPE_F32 ? 4u : 1u);
        if (row_bytes > compiled->widest_row_bytes) compiled->widest_row_bytes = row_bytes;
        compiled->all_rows_bytes += row_bytes;
    }

    for (size_t i = 0; i < plan.count && status == VX_STATUS_OK; i++) {
        const PackagePlan* node = &plan.nodes[i];
        HipStage* stage = &compiled->stages[compiled->stage_count++];
        const char* family = "";
        stage->kind = node->kind;
        stage->input_slot = node->input_slot;
        stage->output_slot = node->output_slot;
        stage->d_in = node->d_in;
        stage->d_out = node->d_out;
        stage->input_dtype = node->input_dtype;
        stage->output_dtype = node->output_dtype;
        if (node->kind == PLAN_PACKED_LINEAR && node->d_in > compiled->widest_float_row)
            compiled->widest_float_row = node->d_in;
        if (node->kind == PLAN_QLINEAR) {
            stage->input_scale = node->input_scale;
            stage->output_scale = node->output_scale;
            stage->input_zero_point = node->input_zero_point;
            stage->output_zero_point = node->output_zero_point;
            status = (VxStatus)vxhip_qlinear_create(node->weight, node->weight_scales, node->weight_zero_points,
                                                    node->bias_i32, node->d_in, node->d_out, node->weight_dtype,
                                                    &stage->qlinear);
            /* a fused integer operator is published only with its multiplier and accumulator-range
             * contract satisfied (docs/w8a8-safetensors.md:158-175, item 8) */
            if (status == VX_STATUS_OK &&
                !vxhip_qlinear_admits(stage->qlinear, node->input_scale, node->input_zero_point, node->output_scale,
                                      node->output_zero_point, (uint32_t)node->input_dtype,
                                      (uint32_t)node->output_dtype))
                status = VX_STATUS_INVALID_GRAPH;
            if (status == VX_STATUS_OK) resident += vxhip_qlinear_resident_bytes(stage->qlinear);
            family = "hip.qlinear";
        } else if (node->kind == PLAN_PACKED_LINEAR) {
            status = (VxStatus)vxhip_packed_linear_create(node->packed_words, node->group_scales, node->bias_f32,
                                                          node->d_in, node->d_out, node->group_size, node->weight_bits,
                                                          &stage->packed);
            if (status == VX_STATUS_OK) resident += vxhip_packed_linear_resident_bytes(stage->packed);
            family = "hip.packed-linear";
        } else if (node->kind == PLAN_REQUANTIZE) {
            stage->input_scale = node->input_scale;
            stage->output_scale = node->output_scale;
            stage->input_zero_point = node->input_zero_point;
            stage->output_zero_point = node->output_zero_point;
            family = "hip.requantize-linear";
        } else {
            stage->input_scale = node->boundary_scale;
            stage->input_zero_point = node->boundary_zero_point;
            family = node->kind == PLAN_QUANTIZE ? "hip.quantize-linear" : "hip.dequantize-linear";
        }
        stage->family = family;
    }
    /* QLinear -> DequantizeLinear with no other reader of the bytes (the tail of a Q / QLinear / DQ
     * sandwich): one launch, no byte tensor */
    for (size_t i = 0; i < compiled->stage_count && status == VX_STATUS_OK; i++) {
        HipStage* linear = &compiled->stages[i];
        size_t readers = 0, reader = 0;
        if (linear->kind != PLAN_QLINEAR) continue;
        for (size_t j = 0; j < compiled->stage_count; j++)
            if (compiled->stages[j].input_slot == linear->output_slot) {
                readers++;
                reader = j;
            }
        for (size_t k = 0; k < compiled->output_count; k++)
            if (compiled->output_slots[k] == linear->output_slot) readers += 2; /* the caller reads the bytes */
        if (readers != 1 || reader <= i || compiled->stages[reader].kind != PLAN_DEQUANTIZE ||
            compiled->stages[reader].input_dtype != linear->output_dtype)
            continue;
        linear->dequantizes = 1;
        linear->dequantized_slot = compiled->stages[reader].output_slot;
        linear->dequantize_scale = compiled->stages[reader].input_scale;
        linear->dequantize_zero_point = compiled->stages[reader].input_zero_point;
        compiled->stages[reader].absorbed = 1;
        linear->family = "hip.qlinear+dequantize-linear";
    }
    /* QuantizeLinear -> QLinear, the bytes read by nobody else and quantized with the linear's input parameters */
    for (size_t i = 0; i < compiled->stage_count && status == VX_STATUS_OK; i++) {
        HipStage* linear = &compiled->stages[i];
        size_t readers = 0, writer = compiled->stage_count;
        if (linear->kind != PLAN_QLINEAR) continue;
        for (size_t j = 0; j < compiled->stage_count; j++) {
            if (compiled->stages[j].input_slot == linear->input_slot) readers++;
            if (compiled->stages[j].output_slot == linear->input_slot) writer = j;
        }
        for (size_t k = 0; k < compiled->output_count; k++)
            if (compiled->output_slots[k] == linear->input_slot) readers += 2;
        if (readers != 1 || writer >= i || compiled->stages[writer].kind != PLAN_QUANTIZE ||
            compiled->stages[writer].output_dtype != linear->input_dtype ||
            memcmp(&compiled->stages[writer].input_scale, &linear->input_scale, sizeof(float)) ||
            compiled->stages[writer].input_zero_point != linear->input_zero_point)
            continue;
        linear->quantizes = 1;
        linear->quantized_slot = compiled->stages[writer].input_slot;
        compiled->stages[writer].absorbed = 1;
        linear->family = linear->dequantizes ? "hip.quantize-linear+qlinear+dequantize-linear" : "hip.quantize-linear+qlinear";
    }
    /* the route names the launches of an execution, in order */
    for (size_t i = 0; i < compiled->stage_count; i++) {
        const HipStage* stage = &compiled->stages[i];
        if (stage->absorbed || !stage->family) continue;
        if (route_used + 1 < sizeof(compiled->route))
            route_used += (size_t)snprintf(compiled->route + route_used, sizeof(compiled->route) - route_used, "%s%s",
                                           route_used ? ">" : "", stage->family);
        if (route_used >= sizeof(compiled->route)) route_used = sizeof(compiled->route) - 1u;
    }
    const int any_packed = plan.any_packed;
    const size_t node_count = plan.count;
    chain_release(&plan);
    if (status != VX_STATUS_OK) {
        fill_report(report, runtime, status, VX_STAGE_COMPILE, code_for(status), vxhip_last_error());
        hip_compiled_destroy(compiled);
        return status;
    }

    for (uint32_t axis = 0; axis + 1 < compiled->rank; axis++) {
        if (rows_max > (UINT64_C(1) << 31) / (uint64_t)compiled->lead_max[axis]) {
            fill_report(report, runtime, VX_STATUS_BACKEND_UNSUPPORTED, VX_STAGE_COMPILE, VX_CODE_BACKEND_UNSUPPORTED,
                        "the bounded domain allows more than 2^31 rows");
            hip_compiled_destroy(compiled);
            return VX_STATUS_BACKEND_UNSUPPORTED;
        }
        rows_max *= (uint64_t)compiled->lead_max[axis];
    }
    attestation->graph_fingerprint = input->graph_fingerprint;
    attestation->shape_domain_proof_identity = input->shape_domain_proof_identity;
    attestation->maximum_tensor_bytes = rows_max * compiled->widest_row_bytes;
    /* weights plus, per context, one buffer per tensor of the graph, the int8 staging of a
     * PackedLinear call (one byte per float of its input, rows padded to 16) and row scales */
    attestation->maximum_resident_bytes = resident + rows_max * (compiled->all_rows_bytes + compiled->widest_float_row + 24u);
    attestation->resource_limit_bytes = 0;
    attestation->has_resource_limit = 0;
    attestation->packed_arithmetic = any_packed ? VX_PACKED_ARITHMETIC_DYNAMIC_I8 : input->packed_arithmetic;
    *out_compiled = compiled;
    fill_report(report, runtime, VX_STATUS_OK, VX_STAGE_COMPILE, VX_CODE_NONE,
                node_count == 1 ? "single-node W8A8 package compiled" : "W8A8 node graph compiled");
    attest(report, compiled->stage_count, compiled->route);
    return VX_STATUS_OK;
}

static void hip_context_destroy(void* context_instance) {
    HipContext* context = (HipContext*)context_instance;
    if (!context) return;
    decoder_state_release(context->decode);
    for (size_t t = 0; t < MAX_GRAPH_TENSORS; t++)
        if (context->tensor_dev[t]) vxhip_device_free(context->tensor_dev[t]);
    for (size_t k = 0; k < MAX_GRAPH_PORTS; k++) free(context->output_host[k]);
    if (context->ctx) vxhip_context_destroy(context->ctx);
    free(context);
}

static VxStatus hip_context_create(void* compiled_instance, const VxContextOptions* options, void** out_context,
                                   VxReport* report) {
    HipCompiled* compiled = (HipCompiled*)compiled_instance;
    HipContext* context;
    VxStatus status;
    if (!out_context) return VX_STATUS_INVALID_ARGUMENT;
    *out_context = NULL;
    if (!compiled || !options || options->struct_size != sizeof(*options)) return VX_STATUS_INVALID_ARGUMENT;
    /* row decode is what a decoder graph offers; a chain of linears has no rows to keep */
    if (options->decode_row_mode != VX_DECODE_ROW_DISABLED &&
        (!compiled->decoder || (options->decode_slots > 1u && options->decode_slots != compiled->decoder->slots)))
        return VX_STATUS_BACKEND_UNSUPPORTED;
    context = (HipContext*)calloc(1, sizeof(*context));
    if (!context) return VX_STATUS_OUT_OF_MEMORY;
    context->compiled = compiled;
    status = (VxStatus)vxhip_context_create(compiled->runtime->device, NULL, VXHIP_CONTEXT_OWN_STREAM, &context->ctx);
    if (status != VX_STATUS_OK) {
        fill_report(report, compiled->runtime, status, VX_STAGE_CONTEXT_CREATE, VX_CODE_BACKEND_CONTEXT_CREATE_FAILED,
                    vxhip_last_error());
        hip_context_destroy(context);
        return status;
    }
    if (compiled->decoder) {
        status = decoder_state_create(compiled->decoder, context->ctx, &context->decode);
        if (status != VX_STATUS_OK) {
            fill_report(report, compiled->runtime, status, VX_STAGE_CONTEXT_CREATE, VX_CODE_BACKEND_CONTEXT_CREATE_FAILED,
                        status == VX_STATUS_OUT_OF_MEMORY ? "the decoder's cache and work buffers do not fit" : vxhip_last_error());
            hip_context_destroy(context);
            return status;
        }
    }
    *out_context = context;
    fill_report(report, compiled->runtime, VX_STATUS_OK, VX_STAGE_CONTEXT_CREATE, VX_CODE_NONE, "context created");
    return VX_STATUS_OK;
}

static VxStatus grow_device(void** buffer, size_t* capacity, size_t bytes) {
    void* fresh = NULL;
    VxStatus status;
    if (bytes <= *capacity) return VX_STATUS_OK;
    status = (VxStatus)vxhip_device_malloc(bytes, &fresh);
    if (status != VX_STATUS_OK) return status;
    if (*buffer) vxhip_device_free(*buffer);
    *buffer = fresh;
    *capacity = bytes;
    return VX_STATUS_OK;
}

static size_t element_bytes(VxDataType dtype) {
    return dtype == VX_DTYPE_F32 ? 4u : 1u;
}

/* Checks the bindings of a call against the compiled contract: every graph input bound exactly
 * once, by name, with its element type, rank, last extent and byte size, all with the same leading
 * extents.  On success the row count, the leading extents and the data pointer of every input. */
static int bindings_admitted(const HipCompiled* compiled, const VxTensorBinding* bindings, size_t binding_count,
                             uint64_t* rows, int64_t* lead, const void** data) {
    *rows = 1;
    if (!bindings || binding_count != compiled->input_count) return 0;
    for (size_t k = 0; k < compiled->input_count; k++) {
        const PlanTensor* t = &compiled->tensors[compiled->input_slots[k]];
        const VxTensorBinding* binding = NULL;
        uint64_t binding_rows = 1;
        for (size_t b = 0; b < binding_count; b++)
            if (bindings[b].struct_size == sizeof(bindings[b]) && bindings[b].name && !strcmp(bindings[b].name, t->name)) {
                if (binding) return 0; /* bound twice */
                binding = &bindings[b];
            }
        if (!binding || binding->dtype != t->dtype || binding->rank != compiled->rank ||
            binding->location != VX_MEMORY_HOST || !binding->data ||
            binding->shape[compiled->rank - 1] != (int64_t)t->d)
            return 0;
        for (uint32_t axis = 0; axis + 1 < compiled->rank; axis++) {
            const int64_t extent = binding->shape[axis];
            if (extent < compiled->lead_min[axis] || extent > compiled->lead_max[axis] ||
                extent % compiled->lead_multiple[axis] != 0 || (k && extent != lead[axis]))
                return 0;
            binding_rows *= (uint64_t)extent;
            lead[axis] = extent;
        }
        if (binding->byte_size != (size_t)binding_rows * t->d * element_bytes(t->dtype)) return 0;
        *rows = binding_rows;
        data[k] = binding->data;
    }
    return 1;
}

/* Upload every input, run every node over all rows (each reads the buffer of its input tensor and
 * writes the buffer of its output tensor), download every graph output into the context's host
 * buffers. */
static VxStatus run_rows(HipContext* context, const void* const* inputs, uint64_t rows, VxReport* report) {
    const HipCompiled* compiled = context->compiled;
    VxStatus status = VX_STATUS_OK;
    for (size_t t = 0; t < compiled->tensor_count && status == VX_STATUS_OK; t++)
        status = grow_device(&context->tensor_dev[t], &context->tensor_capacity[t],
                             (size_t)rows * compiled->tensors[t].d * element_bytes(compiled->tensors[t].dtype));
    for (size_t k = 0; k < compiled->output_count && status == VX_STATUS_OK; k++) {
        const PlanTensor* t = &compiled->tensors[compiled->output_slots[k]];
        const size_t bytes = (size_t)rows * t->d * element_bytes(t->dtype);
        if (bytes > context->host_capacity[k]) {
            void* fresh = realloc(context->output_host[k], bytes);
            if (!fresh) status = VX_STATUS_OUT_OF_MEMORY;
            else {
                context->output_host[k] = fresh;
                context->host_capacity[k] = bytes;
            }
        }
    }
    for (size_t k = 0; k < compiled->input_count && status == VX_STATUS_OK; k++) {
        const PlanTensor* t = &compiled->tensors[compiled->input_slots[k]];
        status = (VxStatus)vxhip_memcpy_to_device(context->ctx, context->tensor_dev[compiled->input_slots[k]], inputs[k],
                                                  (size_t)rows * t->d * element_bytes(t->dtype));
    }
    for (size_t i = 0; i < compiled->stage_count && status == VX_STATUS_OK; i++) {
        const HipStage* stage = &compiled->stages[i];
        const void* from = context->tensor_dev[stage->input_slot];
        void* to = context->tensor_dev[stage->output_slot];
        const uint64_t elements = rows * stage->d_in;
        int handled = 0;
        if (stage->absorbed) continue; /* ran inside the QLinear in front of it */
        switch (stage->kind) {
            case PLAN_QLINEAR:
                if (stage->quantizes)
                    handled = vxhip_qlinear_forward_f32(
                        context->ctx, stage->qlinear, (const float*)context->tensor_dev[stage->quantized_slot],
                        stage->dequantizes ? (float*)context->tensor_dev[stage->dequantized_slot] : NULL,
                        stage->dequantizes ? NULL : to, (uint32_t)rows, stage->input_scale, stage->input_zero_point,
                        stage->output_scale, stage->output_zero_point, (uint32_t)stage->input_dtype,
                        (uint32_t)stage->output_dtype, stage->dequantize_scale, stage->dequantize_zero_point);
                else if (stage->dequantizes)
                    handled = vxhip_qlinear_forward_dequantized(
                        context->ctx, stage->qlinear, from, (float*)context->tensor_dev[stage->dequantized_slot], NULL,
                        (uint32_t)rows, stage->input_scale, stage->input_zero_point, stage->output_scale,
                        stage->output_zero_point, (uint32_t)stage->input_dtype, (uint32_t)stage->output_dtype,
                        stage->dequantize_scale, stage->dequantize_zero_point);
                else
                    handled = vxhip_qlinear_forward(context->ctx, stage->qlinear, from, to, NULL, (uint32_t)rows,
                                                    stage->input_scale, stage->input_zero_point, stage->output_scale,
                                                    stage->output_zero_point, (uint32_t)stage->input_dtype,
                                                    (uint32_t)stage->output_dtype);
                break;
            case PLAN_PACKED_LINEAR:
                handled = vxhip_packed_linear_forward_f32(context->ctx, stage->packed, (const float*)from, (float*)to,
                                                          (uint32_t)rows) == 0;
                break;
            case PLAN_QUANTIZE:
                handled = elements <= UINT32_MAX &&
                          vxhip_quantize_forward(context->ctx, (const float*)from, (uint32_t)elements, to,
                                                 stage->input_scale, stage->input_zero_point,
                                                 (uint32_t)stage->output_dtype);
                break;
            case PLAN_REQUANTIZE:
                handled = elements <= UINT32_MAX &&
                          vxhip_requantize_forward(context->ctx, from, (uint32_t)elements, to, stage->input_scale,
                                                   stage->input_zero_point, stage->output_scale,
                                                   stage->output_zero_point, (uint32_t)stage->input_dtype,
                                                   (uint32_t)stage->output_dtype);
                break;
            case PLAN_DEQUANTIZE:
                handled = elements <= UINT32_MAX &&
                          vxhip_dequantize_forward(context->ctx, from, (uint32_t)elements, stage->input_scale,
                                                   stage->input_zero_point, (uint32_t)stage->input_dtype, (float*)to);
                break;
        }
        if (!handled) status = VX_STATUS_EXECUTION_FAILED;
    }
    for (size_t k = 0; k < compiled->output_count && status == VX_STATUS_OK; k++) {
        const PlanTensor* t = &compiled->tensors[compiled->output_slots[k]];
        status = (VxStatus)vxhip_memcpy_to_host(context->ctx, context->output_host[k],
                                                context->tensor_dev[compiled->output_slots[k]],
                                                (size_t)rows * t->d * element_bytes(t->dtype));
    }
    if (status != VX_STATUS_OK)
        fill_report(report, compiled->runtime, status, VX_STAGE_EXECUTE, code_for(status), vxhip_last_error());
    return status;
}

/* ---- decoder graphs: execute and the decode callbacks ------------------------------------- */

/* The one binding of a decoder graph: the id rows [slots, capacity]. */
static const int32_t* decoder_ids(const DecoderModel* m, const VxTensorBinding* inputs, size_t input_count) {
    const VxTensorBinding* b = inputs;
    if (!inputs || input_count != 1 || b->struct_size != sizeof(*b) || !b->name || strcmp(b->name, m->input_name) ||
        b->dtype != VX_DTYPE_I32 || b->rank != 2 || b->location != VX_MEMORY_HOST || !b->data ||
        b->shape[0] != (int64_t)m->slots || b->shape[1] != (int64_t)m->capacity ||
        b->byte_size != (size_t)m->slots * m->capacity * 4u)
        return NULL;
    return (const int32_t*)b->data;
}

static VxStatus decoder_publish(HipContext* context, const VxBackendOutputSink* sink, VxReport* report, const char* what) {
    const DecoderModel* m = context->compiled->decoder;
    const DecoderState* s = context->decode;
    VxStatus status = VX_STATUS_OK;
    if (m->publish_ids) {
        const int64_t shape[1] = {(int64_t)m->slots};
        status = sink->write(sink->user_data, m->ids_name, VX_DTYPE_I32, shape, 1, s->ids_host, (size_t)m->slots * 4u);
    }
    if (status == VX_STATUS_OK && m->publish_logits) {
        const int64_t shape[2] = {(int64_t)m->slots, (int64_t)m->vocab};
        status = sink->write(sink->user_data, m->logits_name, VX_DTYPE_F32, shape, 2, s->logits_host,
                             (size_t)m->slots * m->vocab * 4u);
    }
    if (status != VX_STATUS_OK) return status;
    fill_report(report, context->compiled->runtime, VX_STATUS_OK, VX_STAGE_EXECUTE, VX_CODE_NONE, what);
    {
        char route[160];
        snprintf(route, sizeof route, "%s%s", vxhip_context_last_variant(context->ctx), s->last_replayed ? "+replay" : "");
        attest(report, m->node_count, route);
    }
    return VX_STATUS_OK;
}

/* Rows first..last through the decoder, then the outputs of row `last`; on success the cache holds
 * rows 0..last.  Everything is validated before the device is touched. */
static VxStatus decoder_rows(HipContext* context, const VxTensorBinding* inputs, size_t input_count, int64_t first,
                             int64_t last, const VxBackendOutputSink* sink, VxReport* report, const char* what) {
    const DecoderModel* m;
    const int32_t* ids;
    VxStatus status;
    if (!context || context->closed || !context->compiled->decoder || !context->decode || !sink ||
        sink->struct_size != sizeof(*sink) || !sink->write)
        return VX_STATUS_INVALID_ARGUMENT;
    m = context->compiled->decoder;
    ids = decoder_ids(m, inputs, input_count);
    if (!ids || first < 0 || last < first || last >= (int64_t)m->capacity) return VX_STATUS_INVALID_ARGUMENT;
    status = decoder_run(m, context->decode, context->ctx, ids, (uint32_t)first, (uint32_t)last);
    if (status != VX_STATUS_OK) {
        context->decode->filled = 0; /* the cache may hold part of the failed call */
        fill_report(report, context->compiled->runtime, status, VX_STAGE_EXECUTE, code_for(status),
                    status == VX_STATUS_INVALID_ARGUMENT ? "a token id lies outside the embedding table" : vxhip_last_error());
        return status;
    }
    context->decode->filled = (int32_t)last + 1;
    return decoder_publish(context, sink, report, what);
}

/* Prefill at `position`: rows 0..position of every slot (native/include/volvoxai_backend.h:214-221). */
static VxStatus hip_context_decode_prefill(void* context_instance, int32_t position, const VxTensorBinding* inputs,
                                           size_t input_count, const VxBackendOutputSink* sink, VxReport* report) {
    HipContext* context = (HipContext*)context_instance;
    if (!context || !context->compiled->decoder) return VX_STATUS_BACKEND_UNSUPPORTED;
    return decoder_rows(context, inputs, input_count, 0, position, sink, report, "W8A8 decoder prefill executed");
}

/* One step: row `position` against the cached rows 0..position-1; the position must be the next
 * unfilled cache slot, else the decode state would no longer describe the rows before it. */
static VxStatus hip_context_decode_step(void* context_instance, int32_t position, const VxTensorBinding* inputs,
                                        size_t input_count, const VxBackendOutputSink* sink, VxReport* report) {
    HipContext* context = (HipContext*)context_instance;
    if (!context || !context->compiled->decoder) return VX_STATUS_BACKEND_UNSUPPORTED;
    if (!context->decode || position < 1 || position != context->decode->filled) return VX_STATUS_INVALID_ARGUMENT;
    return decoder_rows(context, inputs, input_count, position, position, sink, report, "W8A8 decoder step executed");
}

static VxStatus hip_context_decode_reset(void* context_instance, VxReport* report) {
    HipContext* context = (HipContext*)context_instance;
    if (!context || context->closed) return VX_STATUS_INVALID_ARGUMENT;
    if (!context->compiled->decoder) return VX_STATUS_BACKEND_UNSUPPORTED;
    context->decode->filled = 0;
    fill_report(report, context->compiled->runtime, VX_STATUS_OK, VX_STAGE_EXECUTE, VX_CODE_NONE, "decode state reset");
    return VX_STATUS_OK;
}

static VxStatus hip_context_execute(void* context_instance, const VxTensorBinding* inputs, size_t input_count,
                                    const VxBackendOutputSink* sink, VxReport* report) {
    HipContext* context = (HipContext*)context_instance;
    const HipCompiled* compiled;
    int64_t shape[VX_MAX_TENSOR_RANK];
    const void* data[MAX_GRAPH_PORTS];
    uint64_t rows;
    VxStatus status;
    if (!context || context->closed || !inputs || !input_count || !sink || sink->struct_size != sizeof(*sink) ||
        !sink->write)
        return VX_STATUS_INVALID_ARGUMENT;
    compiled = context->compiled;
    if (compiled->decoder) {
        /* the stateless evaluation of a decoder graph: every row, the outputs of the last; no decode
         * state survives it */
        status = decoder_rows(context, inputs, input_count, 0, (int64_t)compiled->decoder->capacity - 1, sink, report,
                              "W8A8 decoder executed");
        context->decode->filled = 0;
        return status;
    }
    /* the complete batch is validated before anything is mutated */
    if (!bindings_admitted(compiled, inputs, input_count, &rows, shape, data)) return VX_STATUS_INVALID_ARGUMENT;
    status = run_rows(context, data, rows, report);
    if (status != VX_STATUS_OK) return status;
    for (size_t k = 0; k < compiled->output_count; k++) {
        const PlanTensor* t = &compiled->tensors[compiled->output_slots[k]];
        shape[compiled->rank - 1] = (int64_t)t->d;
        status = sink->write(sink->user_data, t->name, t->dtype, shape, compiled->rank, context->output_host[k],
                             (size_t)rows * t->d * element_bytes(t->dtype));
        if (status != VX_STATUS_OK) return status;
    }
    fill_report(report, compiled->runtime, VX_STATUS_OK, VX_STAGE_EXECUTE, VX_CODE_NONE, "W8A8 linear executed");
    attest(report, compiled->stage_count, vxhip_context_last_variant(context->ctx));
    return VX_STATUS_OK;
}

/* Frozen batch contract (native/include/volvoxai_backend.h:39-73).  B > 1 is offered along
 * axis 0 only, inside the symbolic range the core handed over and only with its proof identity. */
static VxStatus hip_compiled_batch_contract(void* compiled_instance, VxBackendBatchContract* contract,
                                            VxReport* report) {
    HipCompiled* compiled = (HipCompiled*)compiled_instance;
    if (!compiled || !contract || contract->struct_size != sizeof(*contract)) return VX_STATUS_INVALID_ARGUMENT;
    contract->protocol = VX_BACKEND_BATCH_PROTOCOL;
    contract->resource_domain = compiled;
    contract->compatibility_token = compiled;
    contract->min_batch = 1;
    contract->max_batch = 1;
    contract->multiple_of = 1;
    contract->batch_axis = 0;
    contract->device_resident = 0;
    contract->device_epoch = 0;
    contract->graph_fingerprint = NULL;
    contract->independent_batch_proof_identity = NULL;
    if (compiled->batch_capable && !compiled->decoder) {
        contract->graph_fingerprint = compiled->graph_fingerprint;
        contract->independent_batch_proof_identity = compiled->batch_proof_identity;
        contract->max_batch = compiled->lead_max[0] > 65536 ? 65536u : (uint32_t)compiled->lead_max[0];
    }
    fill_report(report, compiled->runtime, VX_STATUS_OK, VX_STAGE_COMPILE, VX_CODE_NONE, "batch contract frozen");
    return VX_STATUS_OK;
}

/* One entry into the device for the whole invocation: the stacked rows run as one linear and lane
 * i is the i-th slice along axis 0 (native/include/volvoxai_backend.h:75-92). */
static VxStatus hip_context_execute_batch(void* context_instance, const VxBackendBatchInvocation* invocation,
                                          VxReport* report) {
    HipContext* context = (HipContext*)context_instance;
    const HipCompiled* compiled;
    int64_t shape[VX_MAX_TENSOR_RANK];
    const void* data[MAX_GRAPH_PORTS];
    uint64_t rows;
    VxStatus status;
    if (!context || context->closed || !invocation || invocation->struct_size != sizeof(*invocation) ||
        !invocation->stacked_inputs || !invocation->stacked_input_count || !invocation->batch_size ||
        !invocation->lane_output_sinks || invocation->lane_output_sink_count != invocation->batch_size)
        return VX_STATUS_INVALID_ARGUMENT;
    compiled = context->compiled;
    if (compiled->decoder) /* the slots of a decoder are its batch: one invocation, one lane */
        return invocation->batch_size == 1 ? hip_context_execute(context_instance, invocation->stacked_inputs,
                                                                 invocation->stacked_input_count,
                                                                 &invocation->lane_output_sinks[0], report)
                                           : VX_STATUS_BACKEND_UNSUPPORTED;
    if (invocation->batch_size > 1 && !compiled->batch_capable) return VX_STATUS_BACKEND_UNSUPPORTED;
    if (!bindings_admitted(compiled, invocation->stacked_inputs, invocation->stacked_input_count, &rows, shape, data) ||
        shape[0] != (int64_t)invocation->batch_size)
        return VX_STATUS_INVALID_ARGUMENT;
    for (uint32_t lane = 0; lane < invocation->batch_size; lane++) {
        const VxBackendOutputSink* sink = &invocation->lane_output_sinks[lane];
        if (sink->struct_size != sizeof(*sink) || !sink->write) return VX_STATUS_INVALID_ARGUMENT;
    }
    status = run_rows(context, data, rows, report);
    if (status != VX_STATUS_OK) return status;
    shape[0] = 1;
    for (uint32_t lane = 0; lane < invocation->batch_size; lane++) {
        const VxBackendOutputSink* sink = &invocation->lane_output_sinks[lane];
        for (size_t k = 0; k < compiled->output_count; k++) {
            const PlanTensor* t = &compiled->tensors[compiled->output_slots[k]];
            const size_t lane_bytes = (size_t)(rows / invocation->batch_size) * t->d * element_bytes(t->dtype);
            shape[compiled->rank - 1] = (int64_t)t->d;
            status = sink->write(sink->user_data, t->name, t->dtype, shape, compiled->rank,
                                 (const unsigned char*)context->output_host[k] + (size_t)lane * lane_bytes, lane_bytes);
            if (status != VX_STATUS_OK) return status;
        }
    }
    fill_report(report, compiled->runtime, VX_STATUS_OK, VX_STAGE_EXECUTE, VX_CODE_NONE, "W8A8 linear batch executed");
    attest(report, compiled->stage_count, vxhip_context_last_variant(context->ctx));
    return VX_STATUS_OK;
}

static VxStatus hip_context_close(void* context_instance, VxReport* report) {
    HipContext* context = (HipContext*)context_instance;
    (void)report;
    if (!context) return VX_STATUS_INVALID_ARGUMENT;
    context->closed = 1;
    return VX_STATUS_OK;
}

VxStatus volvoxai_hip_gfx950_backend_register(VxReport* report) {
    const VxBackendProvider provider = {
        .struct_size = sizeof(VxBackendProvider),
        .abi_version = VX_BACKEND_ABI_VERSION,
        .name = PROVIDER_NAME,
        .shape_domain = {
            .struct_size = sizeof(VxBackendShapeDomainCapability),
            .proof_protocol = VX_BACKEND_SHAPE_PROOF_PROTOCOL,
            .resource_protocol = VX_BACKEND_RESOURCE_PROTOCOL,
            .support = VX_BACKEND_SHAPE_DOMAIN_FULL,
        },
        .runtime_create = hip_runtime_create,
        .runtime_destroy = hip_runtime_destroy,
        .compile = hip_compile,
        .compiled_destroy = hip_compiled_destroy,
        .compiled_batch_contract = hip_compiled_batch_contract,
        .context_execute_batch = hip_context_execute_batch,
        .context_create = hip_context_create,
        .context_execute = hip_context_execute,
        .context_decode_prefill = hip_context_decode_prefill,
        .context_decode_step = hip_context_decode_step,
        .context_decode_reset = hip_context_decode_reset,
        .context_close = hip_context_close,
        .context_destroy = hip_context_destroy,
        .exact_contract_marker = VX_BACKEND_PROVIDER_EXACT_CONTRACT_MARKER,
        .exact_contract_extent = sizeof(VxBackendProvider),
    };
    return vx_backend_register_provider(&provider, report);
}

/* Reads a package exactly as compile does, without a device: lets a build without a GPU check
 * what the provider would accept.  Returns the compile status and the refusal text. */
VxStatus volvoxai_hip_gfx950_inspect_package(const VxModelSource* source, VxPackedArithmetic arithmetic,
                                             uint32_t* d_in, uint32_t* d_out, int32_t* is_packed_linear,
                                             char* message, size_t message_capacity) {
    ChainPlan plan;
    Failure failure = {VX_STATUS_OK, {0}};
    VxStatus status;
    if (!source || source->struct_size != sizeof(*source)) return VX_STATUS_INVALID_ARGUMENT;
    {
        /* a decoder graph is read by its own route; without a device only the reading is done */
        int is_decoder = 0;
        DecoderModel* unused = NULL;
        status = try_decoder(source, arithmetic, -1, &is_decoder, &unused, &failure);
        if (is_decoder) {
            if (message && message_capacity) snprintf(message, message_capacity, "%s", failure.message);
            if (status == VX_STATUS_OK && is_packed_linear) *is_packed_linear = 1;
            return status;
        }
    }
    status = plan_package(source, arithmetic, &plan, &failure);
    if (message && message_capacity) snprintf(message, message_capacity, "%s", failure.message);
    if (status == VX_STATUS_OK) {
        if (d_in) *d_in = plan.d_in;
        if (d_out) *d_out = plan.d_out;
        if (is_packed_linear) *is_packed_linear = plan.any_packed;
        chain_release(&plan);
    }
    return status;
}
